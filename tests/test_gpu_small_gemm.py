"""Small products whose reduction is dealt to the wavefronts of one block (a block per 32 x 32 tile in fp32, 16 x 16 in
fp64; taken when a problem has far fewer tiles than the chip holds blocks and at most a few dozen reduction steps per
wavefront): dense layers forward and backward with and without a fused activation, convolutions with padding whose input
gradient has few output tiles, a strided input gradient of that size, row and column counts that leave partial tiles,
channel counts around the batch of sixteen steps, against the oracle (fp32 1e-4, fp64 1e-10; DenseKernelLayer.hpp:78-115,
ConvKernelLayer.hpp:125-181)."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}

# batch, inputs, outputs: reductions of one short batch, exactly one batch, several batches with a remainder; outputs that
# leave a partial tile; batches that are not multiples of a tile or of a vector
DENSE = [(256, 784, 512), (256, 512, 256), (256, 256, 10), (128, 1024, 10), (96, 1536, 40), (50, 200, 33), (37, 130, 7),
         (64, 64, 64), (300, 96, 17)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("act", [None, "relu", "tanh", "softplus"])
@pytest.mark.parametrize("case", DENSE, ids=lambda c: "x".join(str(v) for v in c))
def test_dense_layers(case, act, dtype):
    N, K, F = case
    if act in ("tanh", "softplus") and case not in (DENSE[1], DENSE[5]):
        pytest.skip("the other activations on two of the shapes")
    gen = hp.rng(1200 + K + F)
    x = hp.normal(gen, (N, K), dtype)
    w = hp.normal(gen, (K, F), dtype, std=1.0 / np.sqrt(K))
    b = hp.normal(gen, (1, F), dtype)
    g = hp.normal(gen, (N, F), dtype)
    dense = ch.DenseKernelLayer(dtype, (K,), F)
    wp, bp = dense.get_params()
    wp.set_values(w)
    bp.set_values(b)
    layers = [dense]
    if act:
        layers.append(ch.ActivationLayer(dtype, act, (F,)))
    layers = ch.fuse_layers(layers)
    t = ch.DeviceTensor.from_host(x)
    for l in layers:
        t = l.pass_forward(t, True)
    y = t.to_host()
    d = ch.DeviceTensor.from_host(g)
    for l in reversed(layers):
        d = l.pass_back(d)
    dx = d.to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    z_ref = oracle.dense_forward(x64, w64, b64)
    if act:
        y_ref = oracle.act_forward(act, z_ref)
        dz_ref = oracle.act_backward(act, z_ref, y_ref, g64)
    else:
        y_ref, dz_ref = z_ref, g64
    dx_ref, dw_ref, db_ref = oracle.dense_backward(x64, w64, dz_ref)
    tol = TOL[np.dtype(dtype)]
    label = "small gemm dense %s %s %s" % ("x".join(str(v) for v in case), act, np.dtype(dtype).name)
    assert hp.rel_err(y.reshape(y_ref.shape), y_ref, label=label + " y") < tol
    assert hp.rel_err(dx.reshape(dx_ref.shape), dx_ref, label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
    assert hp.rel_err(bp.get_grad(), db_ref) < tol
    # the same pass again: bit for bit
    t = ch.DeviceTensor.from_host(x)
    for l in layers:
        t = l.pass_forward(t, True)
    assert np.array_equal(t.to_host(), y)


# N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh: few output tiles in one or both passes
CONV = [
    (32, 16, 16, 128, 32, 3, 3, 1, 1, 1, 1, 0, 0),       # forward: 8192 x 1152 x 32, the shape of an LSTM's recurrent input gradient
    (32, 16, 16, 32, 128, 3, 3, 1, 1, 1, 1, 0, 0),       # its input gradient is that problem
    (128, 16, 16, 32, 64, 3, 3, 1, 1, 1, 1, 0, 0),       # input gradient 32768 x 576 x 32
    (24, 9, 7, 16, 24, 3, 2, 2, 1, 1, 1, 0, 0),          # padding wider than one, partial tiles in both directions
    (16, 12, 12, 8, 40, 5, 5, 2, 2, 1, 1, 0, 0),         # eight channels: half a batch of steps per tap
    (20, 10, 10, 36, 20, 3, 3, 0, 0, 1, 1, 1, 1),        # dilated receptor, no padding
    (32, 13, 13, 16, 48, 3, 3, 1, 1, 2, 2, 0, 0),        # strided: the input gradient tests divisibility per tap
    (8, 6, 6, 64, 16, 1, 1, 0, 0, 1, 1, 0, 0),           # 1 x 1 receptor
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", CONV, ids=lambda c: "x".join(str(v) for v in c))
def test_convolutions_with_few_tiles(case, dtype):
    N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    geom = dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)
    gen = hp.rng(1300 + H + C + F)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (RH * RW * C, F), dtype, std=1.0 / np.sqrt(RH * RW * C))
    b = hp.normal(gen, (1, F), dtype)
    OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    g = hp.normal(gen, (N, OH, OW, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(g)
    out = layer.pass_forward(xd, True).to_host()
    dx = layer.pass_back(gd).to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
    tol = TOL[np.dtype(dtype)]
    label = "small gemm conv %s %s" % ("x".join(str(v) for v in case), np.dtype(dtype).name)
    assert hp.rel_err(out, o_ref, label=label + " y") < tol
    assert hp.rel_err(dx, dx_ref, label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
    assert hp.rel_err(bp.get_grad(), db_ref) < tol
    layer.pass_forward(xd, True)
    assert np.array_equal(layer.pass_back(gd).to_host(), dx)


def test_non_finite_inputs_stay_where_they_are():
    """Lanes in the padding and steps past the end of a wavefront's share read valid memory and must drop what they read:
    an infinite input element may only reach the outputs whose receptor holds it."""
    dtype = np.float32
    N, H, W, C, F = 32, 8, 8, 32, 32
    geom = dict(RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0)
    gen = hp.rng(1400)
    x = hp.normal(gen, (N, H, W, C), dtype)
    x[0, 0, 0, 0] = np.inf              # element 0 of the tensor: what lanes in the padding read
    x[5, 3, 4, 7] = np.inf
    w = np.abs(hp.normal(gen, (9 * C, F), dtype, std=0.1)) + 0.01
    b = hp.normal(gen, (1, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, 3, 3, 1, 1, 1, 1, 0, 0)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(ch.DeviceTensor.from_host(x), False).to_host()
    ref = oracle.conv_forward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(b, np.float64), **geom)
    assert np.array_equal(np.isfinite(out), np.isfinite(ref))
    assert not np.isnan(out).any()
    fin = np.isfinite(ref)
    assert np.max(np.abs(out[fin] - ref[fin])) < 1e-3


# ---- many tiles in several column blocks: the tiles left over after whole rounds of the chip are cut into parts ------------

@pytest.mark.parametrize("N", [96, 144])
@pytest.mark.parametrize("wide_side", ["forward", "input gradient"])
def test_left_over_tiles_with_several_column_blocks(N, wide_side):
    """Launches whose tiles form more than one column block and do not fill whole rounds of the chip: the left-over rows of
    tiles have their reduction cut into parts that a second launch adds (which batch size leaves such rows depends on how
    many blocks a CU holds, so two are tried). 192 output columns are two column blocks of the widest tile; the wide side
    is the forward pass of a 16 -> 192 layer or the input gradient of a 192 -> 16 layer."""
    dtype = np.float32
    H = W = 28
    C, F = (16, 192) if wide_side == "forward" else (192, 16)
    geom = dict(RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0)
    gen = hp.rng(1500 + N + C)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (9 * C, F), dtype, std=1.0 / np.sqrt(9 * C))
    b = hp.normal(gen, (1, F), dtype)
    g = hp.normal(gen, (N, H, W, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, 3, 3, 1, 1, 1, 1, 0, 0)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(ch.DeviceTensor.from_host(x), True).to_host()
    dx = layer.pass_back(ch.DeviceTensor.from_host(g)).to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
    label = "left-over tiles %s N=%d" % (wide_side, N)
    assert hp.rel_err(out, o_ref, label=label + " y") < 1e-4
    assert hp.rel_err(dx, dx_ref, label=label + " dx") < 1e-4
    assert hp.rel_err(wp.get_grad(), dw_ref) < 1e-4


@pytest.mark.parametrize("case", [(256, 256, 10), (128, 4096, 10), (64, 96, 24), (32, 40, 5)], ids=lambda c: "x".join(str(v) for v in c))
def test_weight_gradient_riding_in_the_input_gradient_launch(case):
    """A last layer's weight gradient (one-wavefront tiles) runs inside its input-gradient launch when both wait for the
    same upstream gradient only. Riding or launched alone (the same layer as a network's first layer, which has no input
    gradient), its slices and their order are the same: the gradients must agree bit for bit, and with the oracle."""
    N, K, F = case
    dtype = np.float32
    gen = hp.rng(1600 + K + F)
    x = hp.normal(gen, (N, K), dtype)
    w = hp.normal(gen, (K, F), dtype, std=1.0 / np.sqrt(K))
    b = hp.normal(gen, (1, F), dtype)
    g = hp.normal(gen, (N, F), dtype)
    grads = []
    for first_layer in (False, True):
        dense = ch.DenseKernelLayer(dtype, (K,), F)
        dense.set_input_layer(first_layer)
        wp, bp = dense.get_params()
        wp.set_values(w)
        bp.set_values(b)
        dense.pass_forward(ch.DeviceTensor.from_host(x), True)
        dx = dense.pass_back(ch.DeviceTensor.from_host(g))
        grads.append((wp.get_grad().copy(), bp.get_grad().copy(), None if first_layer else dx.to_host()))
    assert np.array_equal(grads[0][0], grads[1][0])
    assert np.array_equal(grads[0][1], grads[1][1])
    x64, w64, g64 = (np.asarray(a, np.float64) for a in (x, w, g))
    dx_ref, dw_ref, db_ref = oracle.dense_backward(x64, w64, g64)
    assert hp.rel_err(grads[0][2].reshape(dx_ref.shape), dx_ref, label="riding weight gradient %s dx" % "x".join(str(v) for v in case)) < 1e-4
    assert hp.rel_err(grads[0][0], dw_ref) < 1e-4
    assert hp.rel_err(grads[0][1], db_ref) < 1e-4


@pytest.mark.parametrize("case", [(64, 32, 32, 3, 16, 3, 1), (128, 32, 32, 3, 32, 3, 1), (32, 12, 10, 1, 8, 5, 2), (16, 9, 9, 4, 20, 3, 0),
                                  (12, 8, 8, 2, 6, 3, 1)],
                         ids=lambda c: "x".join(str(v) for v in c))
def test_weight_gradient_riding_in_an_input_gradient_of_few_columns(case):
    """The input gradient of a convolution over one to four channels (no matrix tiles: a lane owns rows and multiplies by
    wave-uniform weights) carries the layer's weight gradient in its launch when that is one of one-wavefront tiles.
    Riding or alone (the same layer as a network's first layer), the weight and bias gradients agree bit for bit; all
    three gradients agree with the oracle. The first two cases are the first layers of BASELINE configs[0] and [2]."""
    N, H, W, C, F, R, pad = case
    dtype = np.float32
    geom = dict(RH=R, RW=R, pv=pad, ph=pad, sv=1, sh=1, dv=0, dh=0)
    gen = hp.rng(1700 + N + F)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (R * R * C, F), dtype, std=1.0 / np.sqrt(R * R * C))
    b = hp.normal(gen, (1, F), dtype)
    OH, OW = hp.conv_dims(H, W, R, R, pad, pad, 1, 1, 0, 0)
    g = hp.normal(gen, (N, OH, OW, F), dtype)
    grads = []
    for first_layer in (False, True):
        layer = ch.ConvKernelLayer(dtype, (H, W, C), F, R, R, pad, pad, 1, 1, 0, 0)
        layer.set_input_layer(first_layer)
        wp, bp = layer.get_params()
        wp.set_values(w)
        bp.set_values(b)
        layer.pass_forward(ch.DeviceTensor.from_host(x), True)
        dx = layer.pass_back(ch.DeviceTensor.from_host(g))
        grads.append((wp.get_grad().copy(), bp.get_grad().copy(), None if first_layer else dx.to_host()))
    assert np.array_equal(grads[0][0], grads[1][0])
    assert np.array_equal(grads[0][1], grads[1][1])
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
    label = "few columns with weight gradient %s" % "x".join(str(v) for v in case)
    assert hp.rel_err(grads[0][2], dx_ref, label=label + " dx") < 1e-4
    assert hp.rel_err(grads[0][0], dw_ref, label=label + " dw") < 1e-4
    assert hp.rel_err(grads[0][1], db_ref.reshape(1, -1), label=label + " db") < 1e-4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", [(32, 16, 16, 8, 128, 3, 1), (16, 10, 12, 5, 7, 3, 1), (8, 9, 9, 6, 6, 5, 2), (12, 8, 8, 40, 8, 3, 0),
                                  (6, 8, 8, 8, 5, 3, 1)],
                         ids=lambda c: "x".join(str(v) for v in c))
def test_five_to_eight_columns_without_matrix_tiles(case, dtype):
    """Products with five to eight output columns (a forward pass with that many filters, an input gradient to that many
    channels) run on the vector ALU like those with up to four when their accesses can be 16 bytes wide. The first case is
    the input-side convolution of BASELINE configs[4] at one time step's batch; the last has a batch that only fp64 can
    take in whole vectors."""
    N, H, W, C, F, R, pad = case
    geom = dict(RH=R, RW=R, pv=pad, ph=pad, sv=1, sh=1, dv=0, dh=0)
    gen = hp.rng(1800 + N + C + F)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (R * R * C, F), dtype, std=1.0 / np.sqrt(R * R * C))
    b = hp.normal(gen, (1, F), dtype)
    OH, OW = hp.conv_dims(H, W, R, R, pad, pad, 1, 1, 0, 0)
    g = hp.normal(gen, (N, OH, OW, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, R, R, pad, pad, 1, 1, 0, 0)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(ch.DeviceTensor.from_host(x), True).to_host()
    dx = layer.pass_back(ch.DeviceTensor.from_host(g)).to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
    tol = 1e-4 if dtype == np.float32 else 1e-10
    label = "five to eight columns %s %s" % ("x".join(str(v) for v in case), np.dtype(dtype).name)
    assert hp.rel_err(out, o_ref, label=label + " y") < tol
    assert hp.rel_err(dx, dx_ref, label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), dw_ref, label=label + " dw") < tol
    assert hp.rel_err(bp.get_grad(), db_ref.reshape(1, -1), label=label + " db") < tol


@pytest.mark.parametrize("case", [(np.float32, 32, 64, 100, 64, 3), (np.float64, 32, 64, 64, 52, 2), (np.float32, 64, 48, 40, 136, 4)],
                         ids=["f32-3", "f64-2", "f32-4"])
def test_few_columns_over_a_large_source(case):
    """A convolution to a few channels whose source is larger than the L2 caches together (the last layer of an image
    decoder) deals its blocks over patches of output positions instead of runs of samples; padding, patch borders and the
    blocks past the last patch must come out as in the plain order. Forward pass against the oracle."""
    dtype, N, H, W, C, F = case
    geom = dict(RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0)
    gen = hp.rng(1900 + C + F)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (9 * C, F), dtype, std=1.0 / np.sqrt(9 * C))
    b = hp.normal(gen, (1, F), dtype)
    assert x.nbytes > 48 << 20
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, 3, 3, 1, 1, 1, 1, 0, 0)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(ch.DeviceTensor.from_host(x), False).to_host()
    ref = oracle.conv_forward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(b, np.float64), **geom)
    tol = 1e-4 if dtype == np.float32 else 1e-10
    assert hp.rel_err(out, ref, label="few columns, large source %s" % "-".join(str(v) for v in case[1:])) < tol


@pytest.mark.parametrize("case", [(np.float32, 32, 32, 32, 64, 3, 3, 1, 1, 0), (np.float32, 24, 40, 36, 30, 4, 4, 2, 1, 0),
                                  (np.float64, 32, 32, 32, 66, 2, 3, 1, 1, 0), (np.float32, 128, 33, 33, 64, 3, 3, 1, 2, 0),
                                  (np.float32, 64, 30, 30, 40, 1, 3, 2, 1, 1), (np.float32, 20, 48, 48, 64, 3, 3, 1, 1, 0)],
                         ids=lambda c: "-".join(str(v) for v in c[1:]))
def test_weight_gradient_of_few_filters(case):
    """The weight and bias gradients of a convolution with up to four filters over many rows (no matrix tiles: a wavefront
    per source channel, sums over lanes at the end of a slice): 3 x 3 and 4 x 4 receptors, a channel count that leaves the
    last block partly empty, stride and dilation, both precisions, and two passes whose gradients accumulate. All three
    gradients against the oracle."""
    dtype, N, H, W, C, F, R, pad, stride, dil = case
    geom = dict(RH=R, RW=R, pv=pad, ph=pad, sv=stride, sh=stride, dv=dil, dh=dil)
    gen = hp.rng(2000 + C + F + R)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (R * R * C, F), dtype, std=1.0 / np.sqrt(R * R * C))
    b = hp.normal(gen, (1, F), dtype)
    OH, OW = hp.conv_dims(H, W, R, R, pad, pad, stride, stride, dil, dil)
    assert N * OH * OW * R * R * C >= 16 << 20
    g = hp.normal(gen, (N, OH, OW, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, R, R, pad, pad, stride, stride, dil, dil)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    for _ in range(2):                      # gradients accumulate until they are reset
        layer.pass_forward(ch.DeviceTensor.from_host(x), True)
        dx = layer.pass_back(ch.DeviceTensor.from_host(g)).to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
    tol = 1e-4 if dtype == np.float32 else 1e-10
    label = "few filters %s" % "-".join(str(v) for v in case[1:])
    assert hp.rel_err(dx, dx_ref, label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), 2 * dw_ref, label=label + " dw") < tol
    assert hp.rel_err(bp.get_grad(), 2 * db_ref.reshape(1, -1), label=label + " db") < tol
