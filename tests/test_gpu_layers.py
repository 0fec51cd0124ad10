"""GPU parity tests: the HIP layers, called through the C ABI, against the CPU oracle on identical
seeded inputs. Tolerances are those of the benchmark definition: fp32 max relative error 1e-4, fp64 1e-10 (metric and
absolute floor in helpers.rel_err), max-pool indices bit-exact."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]


def _tol(dtype):
    return TOL[np.dtype(dtype)]


def _conv_layer(dtype, case):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return ch.ConvKernelLayer(dtype, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)


def _conv_inputs(case, N, dtype, seed):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    g = hp.rng(seed)
    x = hp.uniform(g, (N, H, W, C), -1, 1, dtype)
    w = hp.uniform(g, (RH * RW * C, F), -1, 1, dtype)
    b = hp.uniform(g, (1, F), -1, 1, dtype)
    OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    return x, w, b, go


def _geom(case):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


def _check_conv(case, N, dtype, seed=100):
    x, w, b, go = _conv_inputs(case, N, dtype, seed)
    layer = _conv_layer(dtype, case)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    # truth: the oracle in double precision on the same (already rounded) inputs
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **_geom(case))
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, go64, **_geom(case))
    tol = _tol(dtype)
    assert out.shape == o_ref.shape
    assert hp.rel_err(out, o_ref) < tol, "forward"
    assert hp.rel_err(dx, dx_ref) < tol, "input gradient"
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol, "weight gradient"
    assert hp.rel_err(bp.get_grad(), db_ref) < tol, "bias gradient"
    return layer, (x, w, b, go), (o_ref, dx_ref, dw_ref, db_ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [4, 5])         # 4: vector loads along N; 5: scalar path
@pytest.mark.parametrize("case", hp.REFERENCE_CONV_CASES)
def test_conv_reference_geometries(case, N, dtype):
    _check_conv(case, N, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv_config1_shape(dtype):
    """BASELINE config 1: 64x32x32x3 -> 16 filters 3x3 p1, Glorot-uniform weights, zero bias."""
    case = (32, 32, 3, 16, 3, 3, 1, 1, 1, 1, 0, 0)
    g = hp.rng(0xC0FFEE01)
    N = 64
    x = hp.uniform(g, (N, 32, 32, 3), -1, 1, dtype)
    a = np.sqrt(6.0 / (27 + 16))
    w = hp.uniform(g, (27, 16), -a, a, dtype)
    b = np.zeros((1, 16), dtype)
    go = hp.uniform(g, (N, 32, 32, 16), -1, 1, dtype)
    layer = _conv_layer(dtype, case)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    o_ref, cache = oracle.conv_forward(x, w, b, return_cache=True, **_geom(case))
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w, go, **_geom(case))
    tol = _tol(dtype)
    assert hp.rel_err(out, o_ref) < tol and hp.rel_err(dx, dx_ref) < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol and hp.rel_err(bp.get_grad(), db_ref) < tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv_multi_tile_shape(dtype):
    """Several M tiles per XCD, two F tiles, partial tiles in M, K and F, several wgrad splits."""
    case = (13, 11, 24, 136, 3, 3, 1, 1, 1, 1, 0, 0)
    _check_conv(case, 36, dtype, seed=7)


def test_conv_strided_dilated_larger():
    _check_conv((17, 19, 6, 40, 3, 2, 2, 1, 2, 3, 1, 0), 12, np.float32, seed=8)


@pytest.mark.parametrize("N", [33, 36])              # scalar and 16-byte loads
def test_conv_tall_ragged_problem(N):
    """More than half a million output rows and 40 filters: the 512-row forward tiles that only problems this tall
    use, with partial tiles in M and F."""
    _check_conv((127, 127, 3, 40, 3, 3, 1, 1, 1, 1, 0, 0), N, np.float32, seed=9)


@pytest.mark.parametrize("dtype,N", [(np.float32, 256), (np.float64, 128), (np.float64, 256)])
def test_conv_config4_full_size(dtype, N):
    """BASELINE config 4 at its real shape (56x56x64 -> 128 filters, 3x3 s1 p1; batch 256 in both precisions): the tile
    shapes, left-over-tile splits and weight-gradient slicing that only a problem of this size exercises.
    Checked against the oracle run in the same precision (its own rounding is two orders below the tolerance)
    and, independently of any oracle, through the adjoint identities <conv(x; W), g> = <x, dgrad(g; W)> =
    <W, wgrad(x, g)> and bgrad = sum of g, evaluated in float64 on the GPU's outputs."""
    case = (56, 56, 64, 128, 3, 3, 1, 1, 1, 1, 0, 0)
    g = hp.rng(0xC0FFEE04)
    x = hp.normal(g, (N, 56, 56, 64), dtype)
    w = np.asfortranarray((g.standard_normal((576, 128)) * np.sqrt(2.0 / 576)).astype(dtype))      # He-normal
    b = hp.uniform(g, (1, 128), -0.1, 0.1, dtype)
    go = hp.normal(g, (N, 56, 56, 128), dtype)
    layer = _conv_layer(dtype, case)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    dw, db = wp.get_grad(), bp.get_grad()
    tol = _tol(dtype)
    # adjoint identities (float64 accumulation of the products)
    f64 = np.float64
    lhs = np.vdot(np.asarray(out - b.reshape(1, 1, 1, -1), f64), np.asarray(go, f64))
    scale = np.sqrt(float(np.vdot(np.asarray(out, f64), np.asarray(out, f64))) * float(np.vdot(np.asarray(go, f64), np.asarray(go, f64))))
    assert abs(lhs - np.vdot(np.asarray(x, f64), np.asarray(dx, f64))) < tol * scale * 1e-2
    assert abs(lhs - np.vdot(np.asarray(w, f64), np.asarray(dw, f64))) < tol * scale * 1e-2
    assert hp.rel_err(db.reshape(-1), np.asarray(go, f64).reshape((-1, 128), order="F").sum(axis=0)) < tol
    # the oracle on the same inputs
    o_ref, cache = oracle.conv_forward(x, w, b, return_cache=True, **_geom(case))
    tag = "config 4 %s batch %d " % (np.dtype(dtype).name, N)
    assert hp.rel_err(out, o_ref, label=tag + "forward") < tol
    del out, o_ref
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w, go, **_geom(case))
    assert hp.rel_err(dx, dx_ref, label=tag + "input gradient") < tol
    assert hp.rel_err(dw, dw_ref, label=tag + "weight gradient") < tol
    assert hp.rel_err(db, db_ref, label=tag + "bias gradient") < tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv_accumulates_input_layer_and_clones(dtype):
    case = hp.REFERENCE_CONV_CASES[5]
    layer, (x, w, b, go), (o_ref, dx_ref, dw_ref, db_ref) = _check_conv(case, 8, dtype)
    wp, bp = layer.get_params()
    tol = _tol(dtype)
    # second pass_back accumulates (parameters/StandardParameters.hpp:119); input layers return null
    layer.set_input_layer(True)
    assert layer.is_input_layer()
    assert layer.pass_back(go) is None
    assert hp.rel_err(wp.get_grad(), 2 * dw_ref) < tol and hp.rel_err(bp.get_grad(), 2 * db_ref) < tol
    wp.reset_grad()
    assert not np.any(wp.get_grad())
    # clone_with_shared_params shares values and the gradient accumulator (layer/KernelLayer.hpp:71-77)
    layer.set_input_layer(False)
    twin = layer.clone_with_shared_params()
    bp.reset_grad()
    out2 = twin.pass_forward(x, True)
    assert hp.rel_err(out2, o_ref) < tol
    twin.pass_back(go)
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
    # clone() is a deep copy: new values on the clone leave the original untouched
    deep = layer.clone()
    deep.get_params()[0].set_values(np.zeros_like(w))
    assert np.array_equal(wp.get_values(), np.asfortranarray(w))
    out3 = deep.pass_forward(x, True)
    assert hp.rel_err(out3, np.broadcast_to(np.asarray(b, np.float64).reshape(1, 1, 1, -1), o_ref.shape)) < tol


def test_conv_rank1_and_rank2_views():
    """Rank-1/2 layers are rank-3 layers on re-viewed data (ConvKernelLayer.hpp:400-417, :494-508)."""
    g = hp.rng(9)
    l1 = ch.ConvKernelLayer(np.float64, (32,), 5, 3, 1, 2, 0, 1, 1, 1, 0)
    assert l1.get_output_dims() == (32 * 5,)
    x = hp.normal(g, (3, 32), np.float64)
    w = hp.normal(g, (3, 5), np.float64)
    l1.get_params()[0].set_values(w)
    out = l1.pass_forward(x, True)
    ref = oracle.conv_forward(x.reshape((3, 32, 1, 1), order="F"), w, np.zeros((1, 5)), RH=3, RW=1, pv=2, ph=0, dv=1)
    assert hp.rel_err(out, ref.reshape((3, 32 * 5), order="F")) < 1e-10
    l2 = ch.ConvKernelLayer(np.float64, (10, 10), 5, 3, 2, 1, 2, 1, 2, 1, 0)
    assert l2.get_output_dims() == (8, 7 * 5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,dims,O", [(7, (4, 4, 2), 16), (256, (784,), 512), (33, (40,), 10)])
def test_dense(N, dims, O, dtype):
    g = hp.rng(21)
    V = int(np.prod(dims))
    x = hp.normal(g, (N,) + dims, dtype)
    w = hp.normal(g, (V, O), dtype, std=np.sqrt(2.0 / V))
    b = hp.normal(g, (1, O), dtype)
    go = hp.normal(g, (N, O) + (1,) * (len(dims) - 1), dtype)
    layer = ch.DenseKernelLayer(dtype, dims, O)
    assert layer.get_output_dims() == (O,) + (1,) * (len(dims) - 1)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref = oracle.dense_forward(x64, w64, b64)
    dx_ref, dw_ref, db_ref = oracle.dense_backward(x64, w64, go64.reshape((N, O), order="F"))
    tol = _tol(dtype)
    assert hp.rel_err(out.reshape((N, O), order="F"), o_ref) < tol
    assert hp.rel_err(dx, dx_ref) < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
    assert hp.rel_err(bp.get_grad(), db_ref) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,per_channel", [((16, 8, 8, 6), True), ((128, 16, 16, 8), True), ((9, 4, 4, 2), False),
                                               ((300, 5, 1, 1), False)])
def test_batchnorm(shape, per_channel, dtype):
    g = hp.rng(31)
    x = hp.normal(g, shape, dtype, std=2.0) + dtype(0.5)
    x2 = hp.normal(g, shape, dtype, std=0.7) - dtype(1.0)
    go = hp.normal(g, shape, dtype)
    groups = shape[-1] if per_channel else int(np.prod(shape[1:]))
    gamma = (1 + 0.3 * g.standard_normal(groups)).astype(dtype)
    beta = (0.2 * g.standard_normal(groups)).astype(dtype)
    layer = ch.BatchNormLayer(dtype, shape[1:], norm_avg_decay=0.2, per_last_rank=per_channel)
    params = layer.get_params()
    assert [p.are_optimizable() for p in params] == [False, False, True, True]
    assert np.all(params[2].get_values() == 1) and np.all(params[3].get_values() == 0)
    params[2].set_values(gamma.reshape(1, -1))
    params[3].set_values(beta.reshape(1, -1))
    tol = _tol(dtype)
    # oracle in double on the same inputs
    x64, x264, go64, gamma64, beta64 = (np.asarray(a, np.float64) for a in (x, x2, go, gamma, beta))
    am, ais = np.zeros(groups), np.zeros(groups)
    y_ref, std_ref, isd_ref = oracle.bn_forward(x64, gamma64, beta64, am, ais, False, True, per_channel=per_channel, decay=0.2)
    dx_ref, dg_ref, db_ref = oracle.bn_backward(go64, gamma64, std_ref, isd_ref, per_channel=per_channel)
    assert not layer.stats_initialized()
    y = layer.pass_forward(x, True)
    assert layer.stats_initialized()
    dx = layer.pass_back(go)
    assert hp.rel_err(y, y_ref) < tol
    assert hp.rel_err(dx, dx_ref, label="batchnorm dx %s %s" % (np.dtype(dtype).name, "x".join(map(str, shape)))) < tol
    assert hp.rel_err(params[2].get_grad().reshape(-1), dg_ref) < tol
    assert hp.rel_err(params[3].get_grad().reshape(-1), db_ref) < tol
    assert hp.rel_err(params[0].get_values().reshape(-1), am) < tol
    assert hp.rel_err(params[1].get_values().reshape(-1), ais) < tol
    # second training pass blends the running statistics; inference then uses them
    oracle.bn_forward(x264, gamma64, beta64, am, ais, True, True, per_channel=per_channel, decay=0.2)
    layer.pass_forward(x2, True)
    assert hp.rel_err(params[0].get_values().reshape(-1), am) < tol
    assert hp.rel_err(params[1].get_values().reshape(-1), ais) < tol
    yi_ref, _, _ = oracle.bn_forward(x64, gamma64, beta64, am, ais, True, False, per_channel=per_channel)
    assert hp.rel_err(layer.pass_forward(x, False), yi_ref) < tol
    # input layer: parameter gradients still accumulate, no input gradient
    layer.pass_forward(x, True)
    layer.set_input_layer(True)
    assert layer.pass_back(go) is None
    assert hp.rel_err(params[3].get_grad().reshape(-1), 2 * db_ref) < tol


ACT_CASES = [("identity", 0), ("scaled", 1.7), ("binary_step", 0), ("sigmoid", 0), ("tanh", 0), ("softsign", 0),
             ("softplus", 0), ("relu", 0), ("leaky_relu", 0.1), ("elu", 1.0), ("swish", 1.3)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,p", ACT_CASES)
def test_activations(kind, p, dtype):
    g = hp.rng(41)
    shape = (37, 5, 7, 3)                           # odd element count: exercises the vector tail
    x = hp.normal(g, shape, dtype, std=2.0)
    x[0, 0, 0, 0] = 0
    go = hp.normal(g, shape, dtype)
    layer = ch.ActivationLayer(dtype, kind, shape[1:], p)
    y = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    x64, go64 = np.asarray(x, np.float64), np.asarray(go, np.float64)
    y_ref = oracle.act_forward(kind, x64, float(dtype(p)))
    dx_ref = oracle.act_backward(kind, x64, y_ref, go64, float(dtype(p)))
    tol = _tol(dtype)
    assert hp.rel_err(y, y_ref) < tol
    assert hp.rel_err(dx, dx_ref) < tol
    if kind in ("relu", "leaky_relu", "elu"):
        assert dx[0, 0, 0, 0] == go[0, 0, 0, 0]       # derivative 1 at x == 0
    layer.set_input_layer(True)
    assert layer.pass_back(go) is None


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_prelu_pswish(dtype):
    g = hp.rng(42)
    tol = _tol(dtype)
    N, dims = 70, (10,)
    x = hp.normal(g, (N,) + dims, dtype, std=3.0)
    go = hp.normal(g, (N,) + dims, dtype)
    x64, go64 = np.asarray(x, np.float64), np.asarray(go, np.float64)
    sm = ch.ActivationLayer(dtype, "softmax", dims, 1e-5)
    y = sm.pass_forward(x, True)
    y_ref = oracle.softmax_forward(x64, float(dtype(1e-5)))
    assert hp.rel_err(y, y_ref) < tol
    assert hp.rel_err(sm.pass_back(go), oracle.softmax_backward(y_ref, go64)) < tol
    dims = (3, 4)
    x = hp.normal(g, (N,) + dims, dtype)
    go = hp.normal(g, (N,) + dims, dtype)
    x64, go64 = np.asarray(x, np.float64), np.asarray(go, np.float64)
    for kind, fwd, bwd, init in (("prelu", oracle.prelu_forward, oracle.prelu_backward, 0.1),
                                 ("pswish", oracle.pswish_forward, oracle.pswish_backward, 1.0)):
        layer = ch.ActivationLayer(dtype, kind, dims, init)
        prm = layer.get_params()[0]
        assert prm.get_values().shape == (1, 12) and np.all(prm.get_values() == dtype(init))
        vals = g.uniform(0.05, 1.5, 12).astype(dtype)
        prm.set_values(vals.reshape(1, 12))
        y = layer.pass_forward(x, True)
        dx = layer.pass_back(go)
        v64 = np.asarray(vals, np.float64)
        assert hp.rel_err(y, fwd(x64, v64)) < tol
        dx_ref, pg_ref = bwd(x64, v64, go64)
        assert hp.rel_err(dx, dx_ref) < tol
        assert hp.rel_err(prm.get_grad().reshape(-1), pg_ref) < tol


# the last two: windows that tile the input exactly with a receptor other than 2x2, and a 2x2 pool that leaves
# a row and a column of the input outside every window (their gradient is zero)
POOL_CASES = [(8, 8, 3, 2, 2, 2, 2), (16, 16, 2, 3, 2, 1, 2), (7, 9, 2, 3, 2, 2, 3), (32, 1, 2, 3, 1, 1, 1),
              (32, 32, 32, 2, 2, 2, 2), (9, 8, 2, 3, 2, 3, 2), (9, 9, 2, 2, 2, 2, 2)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [6, 8])                # scalar and 16-byte access paths
@pytest.mark.parametrize("H,W,C,RH,RW,sv,sh", POOL_CASES)
def test_pools(H, W, C, RH, RW, sv, sh, N, dtype):
    g = hp.rng(51)
    x = hp.normal(g, (N, H, W, C), dtype)
    x[:, 0:2, 0, 0] = 3.5                            # ties inside the first window
    mx = ch.MaxPoolLayer(dtype, (H, W, C), RH, RW, sv, sh)
    out = mx.pass_forward(x, True)
    o_ref, i_ref = oracle.maxpool_forward(x, RH, RW, sv, sh)
    assert np.array_equal(out, o_ref)                                  # selection, not arithmetic: exact
    assert np.array_equal(mx.max_indices(N), i_ref)                    # bit-exact argmax cache
    go = hp.normal(g, out.shape, dtype)
    dx = mx.pass_back(go)
    assert np.array_equal(dx, oracle.maxpool_backward(x.shape, go, i_ref, RH, RW, sv, sh))
    mn = ch.MeanPoolLayer(dtype, (H, W, C), RH, RW, sv, sh)
    tol = _tol(dtype)
    assert hp.rel_err(mn.pass_forward(x, True), oracle.meanpool_forward(np.asarray(x, np.float64), RH, RW, sv, sh)) < tol
    assert hp.rel_err(mn.pass_back(go), oracle.meanpool_backward(x.shape, np.asarray(go, np.float64), RH, RW, sv, sh)) < tol
    mx.set_input_layer(True)
    assert mx.pass_back(go) is None


def test_pointwise_layers_at_the_config4_activation_shape():
    """Batch norm, ReLU and both pools on a 256 x 56 x 56 x 64 tensor (51 M elements, the shape the bandwidth
    figures are quoted on): the multi-block reductions and grid-stride loops only a tensor this large exercises."""
    dtype = np.float32
    shape = (256, 56, 56, 64)
    g = hp.rng(61)
    x = hp.normal(g, shape, dtype, std=1.5) + dtype(0.3)
    go = hp.normal(g, shape, dtype)
    x64, go64 = np.asarray(x, np.float64), np.asarray(go, np.float64)
    # batch norm, training pass and backward
    bn = ch.BatchNormLayer(dtype, shape[1:])
    gamma = (1 + 0.2 * g.standard_normal(64)).astype(dtype)
    beta = (0.1 * g.standard_normal(64)).astype(dtype)
    prm = bn.get_params()
    prm[2].set_values(gamma.reshape(1, -1))
    prm[3].set_values(beta.reshape(1, -1))
    am, ais = np.zeros(64), np.zeros(64)
    y_ref, std_ref, isd_ref = oracle.bn_forward(x64, np.asarray(gamma, np.float64), np.asarray(beta, np.float64), am, ais, False, True)
    dx_ref, dg_ref, db_ref = oracle.bn_backward(go64, np.asarray(gamma, np.float64), std_ref, isd_ref)
    assert hp.rel_err(bn.pass_forward(x, True), y_ref) < 1e-4
    assert hp.rel_err(bn.pass_back(go), dx_ref, label="batchnorm dx f32 config-4 activation shape, L = 802,816") < 1e-4
    assert hp.rel_err(prm[2].get_grad().reshape(-1), dg_ref) < 1e-4 and hp.rel_err(prm[3].get_grad().reshape(-1), db_ref) < 1e-4
    assert hp.rel_err(prm[0].get_values().reshape(-1), am) < 1e-4 and hp.rel_err(prm[1].get_values().reshape(-1), ais) < 1e-4
    del y_ref, std_ref, dx_ref
    # ReLU: selection, exact
    relu = ch.ActivationLayer(dtype, "relu", shape[1:])
    assert np.array_equal(relu.pass_forward(x, True), np.maximum(x, 0))
    assert np.array_equal(relu.pass_back(go), np.where(x >= 0, go, dtype(0)))
    # pools: max is a selection (exact, indices bit-exact); mean within tolerance
    gp = hp.normal(g, (256, 28, 28, 64), dtype)
    mx = ch.MaxPoolLayer(dtype, shape[1:])
    o_ref, i_ref = oracle.maxpool_forward(x)
    assert np.array_equal(mx.pass_forward(x, True), o_ref)
    assert np.array_equal(mx.max_indices(256), i_ref)
    assert np.array_equal(mx.pass_back(gp), oracle.maxpool_backward(shape, gp, i_ref))
    mean = ch.MeanPoolLayer(dtype, shape[1:])
    assert hp.rel_err(mean.pass_forward(x, True), oracle.meanpool_forward(x64)) < 1e-4
    assert hp.rel_err(mean.pass_back(gp), oracle.meanpool_backward(shape, np.asarray(gp, np.float64))) < 1e-4


def test_maxpool_nan_and_neg_inf_windows():
    x = np.zeros((1, 4, 4, 1), dtype=np.float32, order="F")
    x[0, 1, 0, 0] = 5
    x[0, 0, 1, 0] = 5
    x[0, 0:2, 2:4, 0] = np.nan
    x[0, 2:4, 0:2, 0] = -np.inf
    x[0, 2, 2, 0] = np.nan
    x[0, 3, 3, 0] = 1
    mx = ch.MaxPoolLayer(np.float32, (4, 4, 1))
    out = mx.pass_forward(x, True)
    o_ref, i_ref = oracle.maxpool_forward(x)
    assert np.array_equal(out, o_ref) and np.array_equal(mx.max_indices(1), i_ref)


def test_device_resident_chain_matches_host_path():
    """conv -> ReLU -> max pool with activations kept in HBM (DeviceTensor) equals the host-tensor path."""
    g = hp.rng(61)
    dtype = np.float32
    N = 8
    x = hp.normal(g, (N, 12, 12, 3), dtype)
    w = hp.normal(g, (27, 8), dtype, std=0.3)
    mk = lambda: (ch.ConvKernelLayer(dtype, (12, 12, 3), 8), ch.ReLUActivationLayer(dtype, (12, 12, 8)),
                  ch.MaxPoolLayer(dtype, (12, 12, 8)))
    host, dev = mk(), mk()
    for conv in (host[0], dev[0]):
        conv.get_params()[0].set_values(w)
    h = x
    for l in host:
        h = l.pass_forward(h, True)
    d = ch.DeviceTensor.from_host(x)
    acts = [d]
    for l in dev:
        acts.append(l.pass_forward(acts[-1], True))
    assert np.array_equal(acts[-1].to_host(), h)
    go = hp.normal(g, h.shape, dtype)
    gh = go
    for l in reversed(host):
        gh = l.pass_back(gh)
    gd = ch.DeviceTensor.from_host(go)
    for l in reversed(dev):
        gd = l.pass_back(gd)
    assert np.array_equal(gd.to_host(), gh)
    assert np.array_equal(dev[0].get_params()[0].get_grad(), host[0].get_params()[0].get_grad())


def test_error_paths():
    """Conditions the reference asserts on become error codes; nothing here launches a bad kernel."""
    with pytest.raises(ch.CattleHipError):
        ch.ConvKernelLayer(np.float32, (4, 4, 1), 0)                       # filters > 0 (ConvKernelLayer.hpp:82)
    with pytest.raises(ch.CattleHipError):
        ch.ConvKernelLayer(np.float32, (2, 2, 1), 1, 5, 5, 0, 0)           # receptor larger than padded input (:86-87)
    with pytest.raises(ch.CattleHipError):
        ch.MaxPoolLayer(np.float32, (2, 2, 1), 3, 3)                       # PoolLayer.hpp:75
    with pytest.raises(ch.CattleHipError):
        ch.BatchNormLayer(np.float32, (4, 4, 2), norm_avg_decay=1.5)       # BatchNormLayer.hpp:80-81
    layer = ch.ConvKernelLayer(np.float32, (4, 4, 1), 2)
    with pytest.raises(ch.CattleHipError) as e:
        layer.pass_back(np.zeros((1, 4, 4, 2), np.float32, order="F"))     # pass_back before pass_forward
    assert e.value.code == 2
    layer.pass_forward(np.zeros((3, 4, 4, 1), np.float32, order="F"), True)
    with pytest.raises(ch.CattleHipError):
        layer.pass_back(np.zeros((2, 4, 4, 2), np.float32, order="F"))     # batch mismatch (ConvKernelLayer.hpp:314)
    with pytest.raises(ValueError):
        layer.pass_forward(np.zeros((3, 5, 4, 1), np.float32, order="F"), True)
    bn = ch.BatchNormLayer(np.float32, (4, 4, 2))
    with pytest.raises(ch.CattleHipError):
        bn.pass_forward(np.zeros((2, 4, 4, 2), np.float32, order="F"), False)   # assert(avgs_init), BatchNormLayer.hpp:245


def test_results_are_reproducible_run_to_run():
    """No atomics anywhere: two identical calls give bit-identical gradients."""
    case = (14, 14, 16, 32, 3, 3, 1, 1, 1, 1, 0, 0)
    x, w, b, go = _conv_inputs(case, 32, np.float32, 77)
    grads = []
    for _ in range(2):
        layer = _conv_layer(np.float32, case)
        layer.get_params()[0].set_values(w)
        layer.pass_forward(x, True)
        dx = layer.pass_back(go)
        grads.append((dx, layer.get_params()[0].get_grad(), layer.get_params()[1].get_grad()))
    for a, b_ in zip(*grads):
        assert np.array_equal(a, b_)
