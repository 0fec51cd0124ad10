"""GPU parity tests of the fused kernel layer (cattle_hip_fused_create): a convolutional or dense layer with the batch
norm, activation and pool layers behind it run as one layer, against the chain of the oracle's *separate* layers in the
order FeedforwardNeuralNetwork.hpp:112-141 calls them. Tolerances: fp32 1e-4, fp64 1e-10 (helpers.rel_err), arg-max
indices bit-exact.

A rectifier or a max pool turns a rounding difference in the convolution output into a different selection, so the
selection tests come in two forms. (a) Inputs, weights and gradients that are multiples of 1/8: every product and sum of
the convolution and of its gradients is then exact in fp32 and fp64 whatever the order of summation, so outputs, arg-max
indices (ties included: they are frequent with such values) and all gradients must equal the oracle's bit for bit.
(b) Random inputs, where the selections of the two sides may differ at near-ties only: indices and rectifier sides are
compared outside a margin around ties, their number inside it is bounded, and gradients are compared with the oracle's
backward chain evaluated on the device's selections."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]
# margin (relative to the RMS of the tensor) inside which two values count as tied for the comparison of selections
MARGIN = {np.dtype(np.float32): 2e-5, np.dtype(np.float64): 1e-12}


def _dyadic(gen, shape, dtype, steps=8):
    return np.asfortranarray(gen.integers(-steps, steps + 1, size=shape).astype(dtype) / steps)


class Chain(object):
    """The oracle's layers behind one another, float64 unless told otherwise: conv/dense, [bn], [act], [pool]."""

    def __init__(self, conv, bn=None, act=None, pool=None, dense=False):
        self.conv, self.bn, self.act, self.pool, self.dense = conv, bn, act, pool, dense

    def forward(self, x, w, b, bn_state=None, training=True):
        c = self.conv
        if self.dense:
            z = oracle.dense_forward(x, w, b)
            self.conv_cache = None
        else:
            z, self.conv_cache = oracle.conv_forward(x, w, b, return_cache=True, **c)
        self.x_shape, self.z = x.shape, z
        cur = z
        if self.bn is not None:
            gamma, beta, avg_mean, avg_inv_sd, init = bn_state
            cur, self.std_cache, self.inv_sd = oracle.bn_forward(cur, gamma, beta, avg_mean, avg_inv_sd, init, training,
                                                                 per_channel=True, decay=self.bn["decay"], eps=self.bn["eps"])
            self.gamma = gamma
        self.pre_act = cur
        if self.act is not None:
            cur = oracle.act_forward(self.act[0], cur, self.act[1])
        self.y = cur
        self.inds = None
        if self.pool is not None:
            kind, RH, RW, sv, sh = self.pool
            if kind == "max":
                cur, self.inds = oracle.maxpool_forward(cur, RH, RW, sv, sh)
            else:
                cur = oracle.meanpool_forward(cur, RH, RW, sv, sh)
        return cur

    def backward(self, x, w, g, inds=None, pre_act=None):
        """inds / pre_act: the selections to differentiate at, if not the chain's own."""
        cur = g
        if self.pool is not None:
            kind, RH, RW, sv, sh = self.pool
            if kind == "max":
                cur = oracle.maxpool_backward(self.y.shape, cur, self.inds if inds is None else inds, RH, RW, sv, sh)
            else:
                cur = oracle.meanpool_backward(self.y.shape, cur, RH, RW, sv, sh)
        if self.act is not None:
            pa = self.pre_act if pre_act is None else pre_act
            cur = oracle.act_backward(self.act[0], pa, oracle.act_forward(self.act[0], pa, self.act[1]), cur, self.act[1])
        grads = {}
        if self.bn is not None:
            cur, grads["gamma"], grads["beta"] = oracle.bn_backward(cur, self.gamma, self.std_cache, self.inv_sd, per_channel=True)
        if self.dense:
            dx, dw, db = oracle.dense_backward(x, w, cur)
        else:
            dx, dw, db = oracle.conv_backward(self.x_shape, self.conv_cache, w, cur, **self.conv)
        grads.update(dx=dx, dw=dw, db=db)
        return grads


def _build(dtype, N, H, W, C, F, conv=None, bn=None, act=None, pool=None, dense=False):
    """Device layers and the fused handle over them; returns (fused, members dict, output dims of the kernel layer)."""
    members = {}
    if dense:
        members["conv"] = ch.DenseKernelLayer(dtype, (H, W, C), F)
        OH, OW = 1, 1
        kdims = (F, 1, 1)
    else:
        g = conv
        members["conv"] = ch.ConvKernelLayer(dtype, (H, W, C), F, g["RH"], g["RW"], g["pv"], g["ph"], g["sv"], g["sh"], g["dv"], g["dh"])
        OH, OW = hp.conv_dims(H, W, g["RH"], g["RW"], g["pv"], g["ph"], g["sv"], g["sh"], g["dv"], g["dh"])
        kdims = (OH, OW, F)
    order = [members["conv"]]
    if bn is not None:
        members["bn"] = ch.BatchNormLayer(dtype, kdims, bn["decay"], bn["eps"], per_last_rank=not dense)
        order.append(members["bn"])
    if act is not None:
        members["act"] = ch.ActivationLayer(dtype, act[0], kdims, act[1])
        order.append(members["act"])
    if pool is not None:
        kind, RH, RW, sv, sh = pool
        cls = ch.MaxPoolLayer if kind == "max" else ch.MeanPoolLayer
        members["pool"] = cls(dtype, kdims, RH, RW, sv, sh)
        order.append(members["pool"])
    return ch.FusedKernelLayer(order), members, kdims


GEOM_3X3 = dict(RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0)


def _run_fused(fused, members, x, w, b, g, bn_vals=None, training=True):
    wp, bp = members["conv"].get_params()
    wp.set_values(w)
    bp.set_values(b)
    if bn_vals is not None:
        ps = members["bn"].get_params()
        ps[2].set_values(bn_vals[0].reshape(1, -1))
        ps[3].set_values(bn_vals[1].reshape(1, -1))
    for q in fused.get_params():
        if q.are_optimizable():
            q.reset_grad()
    out = fused.pass_forward(x, training)
    mode = fused.last_mode()
    dx = fused.pass_back(g) if g is not None else None
    return out, dx, mode


# ---- (a) exact arithmetic: everything bit for bit --------------------------------------------------------------------

EXACT_CASES = [
    # N, H, W, C, F, act, pool, expected mode
    (32, 8, 8, 3, 16, ("relu", 0.0), ("max", 2, 2, 2, 2), "pool"),
    (128, 32, 32, 3, 32, ("relu", 0.0), ("max", 2, 2, 2, 2), "pool"),        # BASELINE config 3, first stage
    (8, 12, 8, 5, 7, ("leaky_relu", 0.125), ("max", 2, 2, 2, 2), "pool"),
    (4, 8, 8, 2, 40, None, ("max", 2, 2, 2, 2), "pool"),
    (64, 16, 16, 4, 8, ("relu", 0.0), ("max", 4, 4, 4, 4), "pool"),
    (16, 8, 8, 3, 6, ("relu", 0.0), ("max", 2, 1, 2, 1), "pool"),
    (16, 9, 9, 3, 6, ("relu", 0.0), None, "act"),
    (256, 4, 4, 6, 5, ("relu", 0.0), ("mean", 2, 2, 2, 2), "pool"),         # mean pooling in the epilogue as well
    (32, 8, 8, 3, 16, None, ("mean", 2, 2, 2, 2), "pool"),
    (64, 16, 16, 4, 8, ("leaky_relu", 0.125), ("mean", 4, 2, 4, 2), "pool"),
    (16, 9, 9, 3, 6, ("relu", 0.0), ("mean", 2, 2, 1, 1), "act"),           # overlapping windows: the pool runs on its own
    (16, 9, 9, 3, 6, ("relu", 0.0), ("max", 3, 3, 2, 2), "act"),            # overlapping windows: the pool runs on its own
    (6, 8, 8, 3, 6, ("relu", 0.0), ("max", 2, 2, 2, 2), None),               # rows of 6: 16-byte accesses in fp64 only
    (7, 8, 8, 3, 6, ("relu", 0.0), ("max", 2, 2, 2, 2), "unfused"),          # rows of 7: member by member
    # tiling windows of more than 64 elements: the pooling epilogue declines, the activation epilogue takes over
    (16, 16, 16, 3, 8, ("relu", 0.0), ("max", 16, 16, 16, 16), "act"),
    (16, 18, 18, 3, 8, ("relu", 0.0), ("max", 9, 9, 9, 9), "act"),
    (16, 16, 16, 3, 8, None, ("max", 8, 16, 8, 16), "unfused"),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", EXACT_CASES)
def test_fused_selections_exact(case, dtype):
    N, H, W, C, F, act, pool, want_mode = case
    gen = hp.rng(7 + N + H)
    x = _dyadic(gen, (N, H, W, C), dtype)
    w = _dyadic(gen, (9 * C, F), dtype)
    b = _dyadic(gen, (1, F), dtype)
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act, pool=pool)
    chain = Chain(GEOM_3X3, act=act, pool=pool)
    ref = chain.forward(*(np.asarray(a, np.float64) for a in (x, w, b)))
    g = _dyadic(gen, ref.shape, dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    if want_mode is None:
        assert mode == "unfused" if np.dtype(dtype) == np.float32 else mode in ("pool", "act")
    else:
        assert mode == want_mode
    grads = chain.backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
    assert np.array_equal(out, ref), "output"
    if pool is not None and pool[0] == "max":
        assert np.array_equal(members["pool"].max_indices(N), chain.inds), "arg-max indices"
    wp, bp = members["conv"].get_params()
    assert np.array_equal(dx, grads["dx"]), "input gradient"
    assert np.array_equal(wp.get_grad(), grads["dw"]), "weight gradient"
    assert np.array_equal(bp.get_grad(), grads["db"].reshape(1, -1)), "bias gradient"


@pytest.mark.parametrize("pool", [("max", 16, 16, 16, 16), ("max", 9, 9, 9, 9), ("max", 2, 2, 2, 2)], ids=lambda p: "%dx%d" % p[1:3])
def test_fused_forward_after_weight_change(pool):
    """The prepared weight layout must follow the weights whichever epilogue a forward pass ends up with: a first pass,
    then an optimizer step on the device, then a second pass, each against the oracle chain on the current weights."""
    dtype, N, C, F = np.float32, 16, 3, 8
    H = W = 18 if pool[1] == 9 else 16
    gen = hp.rng(91)
    x = _dyadic(gen, (N, H, W, C), dtype)
    w = _dyadic(gen, (9 * C, F), dtype)
    b = _dyadic(gen, (1, F), dtype)
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=("relu", 0.0), pool=pool)
    chain = Chain(GEOM_3X3, act=("relu", 0.0), pool=pool)
    wp, bp = members["conv"].get_params()
    for round_ in range(2):
        ref = chain.forward(*(np.asarray(a, np.float64) for a in (x, w, b)))
        g = _dyadic(gen, ref.shape, dtype)
        out, dx, mode = _run_fused(fused, members, x, w, b, g)
        assert mode == ("pool" if pool[1] == 2 else "act")
        grads = chain.backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
        if round_ == 0:
            assert np.array_equal(out, ref), "output"
            assert np.array_equal(members["pool"].max_indices(N), chain.inds)
            assert np.array_equal(dx, grads["dx"])
            assert np.array_equal(wp.get_grad(), grads["dw"])
        else:       # the updated weights are finer-grained: sums may round
            assert hp.rel_err(out, ref, label="fused forward, updated weights") < 1e-5
            assert hp.rel_err(wp.get_grad(), grads["dw"], label="fused dw, updated weights") < 1e-5
        # a step of -1/4 times the (dyadic) gradient keeps the weights dyadic, then one more forward pass on them
        wp.optimizer_update("vanilla_sgd", [0.25])
        w = wp.get_values()
        out2 = fused.pass_forward(x, True)
        ref2 = chain.forward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(b, np.float64))
        assert hp.rel_err(out2, ref2, label="fused forward after update") < 1e-5, "pass after the update %d" % round_


def test_fused_rectifier_side_of_zero():
    """The derivative of ReLU is 1 at an input of exactly zero (x >= 0, ReLUActivationLayer.hpp:51-57) and 0 below; both
    give an output of zero. All-zero weights with a zero bias put every input of the activation at zero."""
    dtype, N, H, W, C, F = np.float32, 16, 8, 8, 3, 4
    gen = hp.rng(3)
    x = _dyadic(gen, (N, H, W, C), dtype)
    for bias, side in ((0.0, 1.0), (-0.5, 0.0)):
        w = np.zeros((9 * C, F), dtype, order="F")
        b = np.full((1, F), bias, dtype, order="F")
        for pool in (None, ("max", 2, 2, 2, 2)):
            fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=("relu", 0.0), pool=pool)
            chain = Chain(GEOM_3X3, act=("relu", 0.0), pool=pool)
            ref = chain.forward(*(np.asarray(a, np.float64) for a in (x, w, b)))
            g = _dyadic(gen, ref.shape, dtype)
            out, dx, mode = _run_fused(fused, members, x, w, b, g)
            assert mode == ("pool" if pool else "act")
            assert np.array_equal(out, ref) and not np.any(out)
            grads = chain.backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
            assert np.array_equal(members["conv"].get_params()[1].get_grad(), grads["db"].reshape(1, -1))
            assert np.array_equal(members["conv"].get_params()[0].get_grad(), grads["dw"])
            assert (np.abs(grads["db"]).sum() > 0) == (side > 0)


# ---- (b) random inputs -----------------------------------------------------------------------------------------------

def _compare_selections(chain, dev_inds, dtype, pool):
    """Arg-max indices equal the oracle's except in windows whose two largest values are within the margin; returns
    the share of windows that differ."""
    if dev_inds is None:
        return 0.0
    differ = dev_inds != chain.inds
    if not differ.any():
        return 0.0
    kind, RH, RW, sv, sh = pool
    y = chain.y
    N, H, W, C = y.shape
    OH, OW = oracle.pool_out_dims(H, W, RH, RW, sv, sh)
    margin = MARGIN[np.dtype(dtype)] * float(np.sqrt(np.mean(y * y)))
    pos, col = np.nonzero(differ)
    for p, cn in zip(pos, col):
        ow, oh = divmod(int(p), OH)
        c, n = divmod(int(cn), N)
        win = y[n, oh * sv:oh * sv + RH, ow * sh:ow * sh + RW, c]
        a, b_ = int(dev_inds[p, cn]), int(chain.inds[p, cn])
        va, vb = win[a % RH, a // RH], win[b_ % RH, b_ // RH]
        assert abs(va - vb) <= margin, "arg-max differs outside the tie margin"
    return differ.mean()


def _argmax_positions(inds, N, H, W, C, pool):
    """Index arrays (n, h, w, c) of the selected element of every window, and (n, oh, ow, c) of the window."""
    kind, RH, RW, sv, sh = pool
    OH, OW = oracle.pool_out_dims(H, W, RH, RW, sv, sh)
    pos, col = np.meshgrid(np.arange(OH * OW), np.arange(C * N), indexing="ij")
    ow, oh = np.divmod(pos, OH)
    c, n = np.divmod(col, N)
    k, l = np.divmod(inds.astype(np.int64), RH)
    return (n, oh * sv + l, ow * sh + k, c), (n, oh, ow, c)


def _pre_act_at_device_sides(chain, dev_out, dev_inds, dtype):
    """The oracle's activation input with the sign of those elements turned whose side of the rectifier's kink differs
    from the one the device's output shows: allowed within the margin of zero only, and rarely."""
    if chain.act is None or chain.act[0] not in ("relu", "leaky_relu", "elu") or chain.act[1] < 0:
        return None
    if chain.pool is not None and chain.pool[0] != "max":
        return None
    pa = chain.pre_act
    margin = MARGIN[np.dtype(dtype)] * float(np.sqrt(np.mean(pa * pa)))
    dev_out = np.asarray(dev_out, np.float64)
    if chain.pool is None:
        dev_out = dev_out.reshape(pa.shape, order="F")
    pre = pa.copy(order="F")
    if chain.pool is None:
        flipped = (dev_out > 0) != (pa > 0)
        assert np.all(np.abs(pa[flipped]) <= margin), "rectifier side differs outside the margin"
        pre[flipped] = -pa[flipped]
        share = flipped.mean()
    else:
        N, H, W, C = pa.shape
        full, pooled = _argmax_positions(dev_inds, N, H, W, C, chain.pool)
        at = pa[full]
        flipped = (dev_out[pooled] > 0) != (at > 0)
        assert np.all(np.abs(at[flipped]) <= margin), "rectifier side differs outside the margin"
        fi = tuple(a[flipped] for a in full)
        pre[fi] = -pa[fi]
        share = flipped.mean()
    assert share < 1e-3
    return pre


def _kink_free(z, dtype):
    """No value within the margin of zero (for activations whose output does not show the side of the input)."""
    return float(np.min(np.abs(z))) > MARGIN[np.dtype(dtype)] * float(np.sqrt(np.mean(z * z)))


SMOOTH_ACTS = [("sigmoid", 0.0), ("tanh", 0.0), ("softplus", 0.0), ("swish", 1.25), ("softsign", 0.0), ("elu", 0.75),
               ("scaled", 1.5), ("identity", 0.0), ("leaky_relu", -0.25), ("elu", -0.5), ("binary_step", 0.0)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", SMOOTH_ACTS, ids=lambda a: "%s-%g" % a)
@pytest.mark.parametrize("pooled", [False, True])
def test_fused_activations(act, pooled, dtype):
    N, H, W, C, F = 32, 8, 12, 5, 20
    pool = ("max", 2, 2, 2, 2) if pooled else None
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act, pool=pool)
    chain = Chain(GEOM_3X3, act=act, pool=pool)
    hidden_side = act[0] in ("leaky_relu", "elu") and act[1] < 0        # positive outputs on both sides of the kink
    for seed in range(11, 31):
        gen = hp.rng(seed)
        x = hp.uniform(gen, (N, H, W, C), -1, 1, dtype)
        w = hp.uniform(gen, (9 * C, F), -0.4, 0.4, dtype)
        b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
        x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
        ref = chain.forward(x64, w64, b64)
        if not hidden_side or _kink_free(chain.z, dtype):
            break
    else:
        pytest.fail("no seed gives inputs that stay clear of the kink")
    g = hp.uniform(gen, ref.shape, -1, 1, dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    assert mode == ("pool" if pooled else "act")
    tol = TOL[np.dtype(dtype)]
    label = "fused %s%s %s" % (act[0], " pool" if pooled else "", np.dtype(dtype).name)
    if act[0] == "binary_step":
        assert np.mean(np.asarray(out, np.float64) != ref) < 1e-4
    else:
        assert hp.rel_err(out, ref, label=label + " forward") < tol
    dev_inds = members["pool"].max_indices(N) if pooled else None
    assert _compare_selections(chain, dev_inds, dtype, pool) < 1e-3
    grads = chain.backward(x64, w64, np.asarray(g, np.float64), inds=dev_inds, pre_act=_pre_act_at_device_sides(chain, out, dev_inds, dtype))
    wp, bp = members["conv"].get_params()
    assert hp.rel_err(dx, grads["dx"], label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), grads["dw"], label=label + " dw") < tol
    assert hp.rel_err(bp.get_grad(), grads["db"].reshape(1, -1), label=label + " db") < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", [None, ("relu", 0.0), ("sigmoid", 0.0), ("tanh", 0.0), ("softplus", 0.0), ("swish", 1.25),
                                 ("scaled", 1.5), ("elu", 0.75), ("leaky_relu", -0.25)], ids=lambda a: "none" if a is None else "%s-%g" % a)
@pytest.mark.parametrize("window", [(2, 2), (2, 4), (4, 4)], ids=lambda w: "%dx%d" % w)
def test_fused_mean_pool_epilogue(act, window, dtype):
    """conv -> [activation] -> mean pool whose windows tile the output (MeanPoolLayer.hpp:35-47): the means come out of the
    GEMM's epilogue, the backward pass spreads g / window size over every position times the activation's derivative
    there, read from what the forward pass kept (coded outputs, or inputs for kinds whose derivative needs them)."""
    prh, prw = window
    N, H, W, C, F = 32, 12, 8, 5, 20
    pool = ("mean", prh, prw, prh, prw)
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act, pool=pool)
    chain = Chain(GEOM_3X3, act=act, pool=pool)
    hidden_side = act is not None and act[0] in ("leaky_relu", "elu") and act[1] < 0
    for seed in range(50, 70):
        gen = hp.rng(seed)
        x = hp.uniform(gen, (N, H, W, C), -1, 1, dtype)
        w = hp.uniform(gen, (9 * C, F), -0.4, 0.4, dtype)
        b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
        x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
        ref = chain.forward(x64, w64, b64)
        if not hidden_side or _kink_free(chain.z, dtype):
            break
    else:
        pytest.fail("no seed gives inputs that stay clear of the kink")
    g = hp.uniform(gen, ref.shape, -1, 1, dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    assert mode == "pool"
    tol = TOL[np.dtype(dtype)]
    label = "fused %s mean pool %dx%d %s" % ("none" if act is None else act[0], prh, prw, np.dtype(dtype).name)
    assert hp.rel_err(out, ref, label=label + " forward") < tol
    # the rectifier's side where the device's pre-activation value rounds to the other side of zero: rare, and only
    # within the margin, so the gradient comparison allows for the few elements it moves
    grads = chain.backward(x64, w64, np.asarray(g, np.float64))
    wp, bp = members["conv"].get_params()
    near_kink = act is not None and act[0] in ("relu", "leaky_relu", "elu") and not _kink_free(chain.z, dtype)
    if near_kink:
        pytest.skip("an input within the tie margin of the rectifier's kink: covered by the exact-arithmetic cases")
    assert hp.rel_err(dx, grads["dx"], label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), grads["dw"], label=label + " dw") < tol
    assert hp.rel_err(bp.get_grad(), grads["db"].reshape(1, -1), label=label + " db") < tol


BN = dict(decay=0.1, eps=1e-5)
BN_CASES = [
    # N, H, W, C, F, act, pool, dense
    (128, 16, 16, 32, 64, ("relu", 0.0), ("max", 2, 2, 2, 2), False),       # BASELINE config 3, second stage
    (16, 8, 8, 3, 6, None, None, False),
    (16, 8, 8, 3, 6, ("sigmoid", 0.0), ("mean", 2, 2, 2, 2), False),
    (32, 6, 10, 4, 9, ("tanh", 0.0), ("max", 2, 2, 2, 2), False),
    (8, 9, 9, 3, 5, ("softplus", 0.0), ("max", 3, 3, 2, 2), False),          # overlapping windows behind the chain pass
    (64, 1, 1, 48, 24, ("relu", 0.0), None, True),
    # more than a thousand GEMM tiles: their moments are merged by a launch of its own in front of the chain's forward pass
    (64, 96, 96, 3, 8, ("relu", 0.0), ("max", 2, 2, 2, 2), False),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", BN_CASES)
def test_fused_batch_norm_chain(case, dtype):
    N, H, W, C, F, act, pool, dense = case
    gen = hp.rng(23 + N)
    x = hp.normal(gen, (N, H, W, C), dtype)
    K = H * W * C if dense else 9 * C
    w = hp.normal(gen, (K, F), dtype, std=float(np.sqrt(2.0 / K)))
    b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
    gamma = hp.uniform(gen, (F,), 0.5, 1.5, dtype)
    beta = hp.uniform(gen, (F,), -0.5, 0.5, dtype)
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, bn=BN, act=act, pool=pool, dense=dense)
    chain = Chain(GEOM_3X3, bn=BN, act=act, pool=pool, dense=dense)
    x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
    avg_mean, avg_inv_sd = np.zeros(F), np.zeros(F)
    tol = TOL[np.dtype(dtype)]
    label = "fused bn %s %s %s" % (act[0] if act else "-", pool[0] if pool else "-", np.dtype(dtype).name)
    init = False
    for step in range(2):          # the first pass assigns the running statistics, the second averages them
        ref = chain.forward(x64 + step, w64, b64, bn_state=(np.asarray(gamma, np.float64), np.asarray(beta, np.float64), avg_mean,
                                                             avg_inv_sd, init), training=True)
        init = True
        g = hp.uniform(gen, ref.shape, -1, 1, dtype)
        out, dx, mode = _run_fused(fused, members, np.asfortranarray((x + step).astype(dtype)), w, b,
                                   g.reshape((N,) + fused.get_output_dims(), order="F"), bn_vals=(gamma, beta))
        out = out.reshape(ref.shape, order="F")
        assert mode == "bn"
        assert hp.rel_err(out, ref, label=label + " forward") < tol
        ps = members["bn"].get_params()
        assert hp.rel_err(ps[0].get_values().ravel(), avg_mean, label=label + " running mean") < tol
        assert hp.rel_err(ps[1].get_values().ravel(), avg_inv_sd, label=label + " running inv sd") < tol
        assert members["bn"].stats_initialized()
        tiling_max = pool is not None and pool[0] == "max"
        dev_inds = members["pool"].max_indices(N) if tiling_max else None
        assert _compare_selections(chain, dev_inds, dtype, pool) < 1e-3
        grads = chain.backward(x64 + step, w64, np.asarray(g, np.float64), inds=dev_inds,
                               pre_act=_pre_act_at_device_sides(chain, out, dev_inds, dtype))
        wp, bp = members["conv"].get_params()
        btol = tol
        assert hp.rel_err(ps[2].get_grad().ravel(), grads["gamma"], label=label + " dgamma") < btol
        assert hp.rel_err(ps[3].get_grad().ravel(), grads["beta"], label=label + " dbeta") < btol
        assert hp.rel_err(dx, grads["dx"], label=label + " dx") < btol
        assert hp.rel_err(wp.get_grad(), grads["dw"], label=label + " dw") < btol
    # inference from the running statistics
    ref = chain.forward(x64, w64, b64, bn_state=(np.asarray(gamma, np.float64), np.asarray(beta, np.float64), avg_mean, avg_inv_sd,
                                                 True), training=False)
    out = fused.pass_forward(x, False).reshape(ref.shape, order="F")
    assert fused.last_mode() == "bn"
    assert hp.rel_err(out, ref, label=label + " inference") < tol
    with pytest.raises(ch.CattleHipError) as e:
        fused.pass_back(g.reshape((N,) + fused.get_output_dims(), order="F"))
    assert e.value.code == 2


def test_fused_dense_relu_exact():
    """DenseKernelLayer -> ReLU (BASELINE config 2's hidden layers) with exact arithmetic."""
    for dtype in DTYPES:
        N, V, F = 256, 96, 40
        gen = hp.rng(5)
        x = _dyadic(gen, (N, V, 1, 1), dtype)
        w = _dyadic(gen, (V, F), dtype)
        b = _dyadic(gen, (1, F), dtype)
        fused, members, kdims = _build(dtype, N, V, 1, 1, F, act=("relu", 0.0), dense=True)
        chain = Chain(None, act=("relu", 0.0), dense=True)
        ref = chain.forward(*(np.asarray(a, np.float64) for a in (x, w, b)))
        g = _dyadic(gen, ref.shape, dtype)
        out, dx, mode = _run_fused(fused, members, x, w, b, g.reshape((N,) + fused.get_output_dims(), order="F"))
        assert mode == "act"
        grads = chain.backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
        assert np.array_equal(out.reshape(ref.shape, order="F"), ref)
        assert np.array_equal(dx.reshape(grads["dx"].shape), grads["dx"])
        assert np.array_equal(members["conv"].get_params()[0].get_grad(), grads["dw"])


def test_fused_unfusable_members_run_one_by_one():
    """Softmax and PReLU cannot be an epilogue: the handle still equals the chain, member by member."""
    dtype, N, V, F = np.float64, 16, 12, 10
    gen = hp.rng(9)
    x = hp.uniform(gen, (N, V), -1, 1, dtype)
    w = hp.uniform(gen, (V, F), -1, 1, dtype)
    b = hp.uniform(gen, (1, F), -1, 1, dtype)
    dense = ch.DenseKernelLayer(dtype, (V,), F)
    soft = ch.ActivationLayer(dtype, "softmax", (F,), 1e-5)
    fused = ch.FusedKernelLayer([dense, soft])
    dense.get_params()[0].set_values(w)
    dense.get_params()[1].set_values(b)
    out = fused.pass_forward(x, True)
    assert fused.last_mode() == "unfused"
    z = oracle.dense_forward(x, w, b)
    y = oracle.softmax_forward(z)
    assert hp.rel_err(out, y) < 1e-10
    g = hp.uniform(gen, y.shape, -1, 1, dtype)
    dx = fused.pass_back(g)
    dz = oracle.softmax_backward(y, g)
    dx_ref, dw_ref, db_ref = oracle.dense_backward(x, w, dz)
    assert hp.rel_err(dx, dx_ref) < 1e-10
    assert hp.rel_err(dense.get_params()[0].get_grad(), dw_ref) < 1e-10


def test_fused_handle_shares_parameters_and_guards_state():
    dtype, N, H, W, C, F = np.float32, 16, 8, 8, 3, 6
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, bn=BN, act=("relu", 0.0), pool=("max", 2, 2, 2, 2))
    ps = fused.get_params()
    assert len(ps) == 2 + 4
    assert [q.are_optimizable() for q in ps] == [True, True, False, False, True, True]
    gen = hp.rng(1)
    w = hp.uniform(gen, (9 * C, F), -1, 1, dtype)
    ps[0].set_values(w)
    assert np.array_equal(members["conv"].get_params()[0].get_values(), w)       # the same parameter object
    assert fused.get_output_dims() == (4, 4, F)
    g = hp.uniform(gen, (N, 4, 4, F), -1, 1, dtype)
    with pytest.raises(ch.CattleHipError) as e:
        fused.pass_back(g)
    assert e.value.code == 2
    x = hp.uniform(gen, (N, H, W, C), -1, 1, dtype)
    fused.pass_forward(x, True)
    fused.empty_cache()
    with pytest.raises(ch.CattleHipError) as e:
        fused.pass_back(g)
    assert e.value.code == 2
    # a wrong order of members is refused
    with pytest.raises(ch.CattleHipError):
        ch.FusedKernelLayer([members["act"], members["conv"]])
    # a clone owns clones of the members and gives the same result
    out = fused.pass_forward(x, True)
    clone = fused.clone()
    out_c = clone.pass_forward(x, False)          # from the running statistics the clone copied
    out_i = fused.pass_forward(x, False)
    assert np.array_equal(out_c, out_i)
    assert out.shape == out_c.shape


def test_fused_input_layer_skips_the_input_gradient():
    dtype, N, H, W, C, F = np.float32, 16, 8, 8, 3, 6
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=("relu", 0.0), pool=("max", 2, 2, 2, 2))
    fused.set_input_layer(True)
    gen = hp.rng(2)
    x = _dyadic(gen, (N, H, W, C), dtype)
    w = _dyadic(gen, (9 * C, F), dtype)
    b = _dyadic(gen, (1, F), dtype)
    g = _dyadic(gen, (N, 4, 4, F), dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    assert dx is None and mode == "pool"
    chain = Chain(GEOM_3X3, act=("relu", 0.0), pool=("max", 2, 2, 2, 2))
    chain.forward(*(np.asarray(a, np.float64) for a in (x, w, b)))
    grads = chain.backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
    assert np.array_equal(members["conv"].get_params()[0].get_grad(), grads["dw"])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", [("relu", 0.0), ("leaky_relu", 0.125), ("elu", 0.5), None, ("tanh", 0.0)])
@pytest.mark.parametrize("window", [(2, 2), (4, 2), (1, 2), (3, 3)])
def test_first_layer_weight_gradient_from_the_pooled_gradient(window, act, dtype):
    """A fused first layer (nobody needs its input gradient) with a rectifier or no activation and a max pool whose window
    sides are powers of two forms the gradient of the convolution output inside the weight-gradient launch, from the pooled
    gradient, the arg-max cache and the coded outputs; the pass that scatters it does not run. The gradients must equal, bit
    for bit, those of the same layer when it is not the first (where that pass runs), and agree with the oracle's chain.
    Other activations and windows (3 x 3) take the usual path either way."""
    prh, prw = window
    N, H, W, C, F = 16, 12, 12, 3, 10
    pool = ("max", prh, prw, prh, prw)
    gen = hp.rng(77 + prh * 8 + prw)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (9 * C, F), dtype, std=0.3)
    b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
    g = hp.normal(gen, (N, H // prh, W // prw, F), dtype)
    runs = []
    for first in (False, True):
        fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act, pool=pool)
        fused.set_input_layer(first)
        out, dx, mode = _run_fused(fused, members, x, w, b, g)
        assert mode == "pool" or window == (3, 3)
        assert (dx is None) == first or mode == "unfused"
        wp, bp = members["conv"].get_params()
        runs.append((wp.get_grad().copy(), bp.get_grad().copy(), members["pool"].max_indices(N), out))
    assert np.array_equal(runs[0][0], runs[1][0])
    assert np.array_equal(runs[0][1], runs[1][1])
    assert np.array_equal(runs[0][2], runs[1][2])
    dw, db, dev_inds, out = runs[1]
    chain = Chain(GEOM_3X3, act=act, pool=pool)
    x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
    chain.forward(x64, w64, b64)
    assert _compare_selections(chain, dev_inds, dtype, pool) < 1e-3
    ref = chain.backward(x64, w64, np.asarray(g, np.float64), inds=dev_inds,
                         pre_act=_pre_act_at_device_sides(chain, out, dev_inds, dtype))
    tol = TOL[np.dtype(dtype)]
    label = "first layer %dx%d %s %s" % (prh, prw, act[0] if act else "-", np.dtype(dtype).name)
    assert hp.rel_err(dw, ref["dw"], label=label + " dw") < tol
    assert hp.rel_err(db, ref["db"].reshape(1, -1), label=label + " db") < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [6, 7, 2, 36])
def test_first_layer_weight_gradient_with_ragged_batches(N, dtype):
    """Batches that are not whole 16-byte vectors of samples (or only in fp64) take the path with the scatter pass; a first
    layer's gradients must not depend on which path ran."""
    H, W, C, F = 8, 8, 3, 6
    act, pool = ("relu", 0.0), ("max", 2, 2, 2, 2)
    gen = hp.rng(900 + N)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (9 * C, F), dtype, std=0.3)
    b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
    g = hp.normal(gen, (N, H // 2, W // 2, F), dtype)
    runs = []
    for first in (False, True):
        fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act, pool=pool)
        fused.set_input_layer(first)
        out, dx, mode = _run_fused(fused, members, x, w, b, g)
        wp, bp = members["conv"].get_params()
        runs.append((wp.get_grad().copy(), bp.get_grad().copy(), mode))
    assert runs[0][2] == runs[1][2]
    assert np.array_equal(runs[0][0], runs[1][0])
    assert np.array_equal(runs[0][1], runs[1][1])
    chain = Chain(GEOM_3X3, act=act, pool=pool)
    x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
    chain.forward(x64, w64, b64)
    ref = chain.backward(x64, w64, np.asarray(g, np.float64))
    tol = TOL[np.dtype(dtype)]
    assert hp.rel_err(runs[1][0], ref["dw"], label="first layer N=%d %s dw" % (N, np.dtype(dtype).name)) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("F", [1, 3, 4, 6, 8])
@pytest.mark.parametrize("act", [("tanh", 0.0), ("sigmoid", 0.0), ("relu", 0.0), ("leaky_relu", 0.125), ("softplus", 0.0)],
                         ids=lambda a: a[0])
def test_fused_activation_behind_a_few_filters(act, F, dtype):
    """A kernel layer with one to eight filters and its activation as one fused layer (the output layer of an image decoder):
    the product runs without matrix tiles and applies the activation as it stores. Forward and all gradients against the
    oracle's layers behind one another."""
    N, H, W, C = 16, 12, 10, 24
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=GEOM_3X3, act=act)
    chain = Chain(GEOM_3X3, act=act)
    gen = hp.rng(300 + F)
    x = hp.uniform(gen, (N, H, W, C), -1, 1, dtype)
    w = hp.uniform(gen, (9 * C, F), -0.3, 0.3, dtype)
    b = hp.uniform(gen, (1, F), -0.5, 0.5, dtype)
    x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
    ref = chain.forward(x64, w64, b64)
    g = hp.uniform(gen, ref.shape, -1, 1, dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    assert mode == "act"
    tol = TOL[np.dtype(dtype)]
    label = "fused %s behind %d filters %s" % (act[0], F, np.dtype(dtype).name)
    assert hp.rel_err(out, ref, label=label + " forward") < tol
    grads = chain.backward(x64, w64, np.asarray(g, np.float64), pre_act=_pre_act_at_device_sides(chain, out, None, dtype))
    wp, bp = members["conv"].get_params()
    assert hp.rel_err(dx, grads["dx"], label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), grads["dw"], label=label + " dw") < tol
    assert hp.rel_err(bp.get_grad(), grads["db"].reshape(1, -1), label=label + " db") < tol


# ---- a seeded sweep of fused groups over geometries nobody chose by hand ------------------------------------------------

def _sweep_cases(count, seed):
    g = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        RH, RW = int(g.integers(1, 4)), int(g.integers(1, 4))
        dv, dh = int(g.integers(0, 2)), int(g.integers(0, 2))
        sv, sh = int(g.integers(1, 3)), int(g.integers(1, 3))
        pv, ph = int(g.integers(0, RH)), int(g.integers(0, RW))
        H, W = int(g.integers(2, 34)), int(g.integers(2, 34))
        eh, ew = (RH - 1) * (dv + 1) + 1, (RW - 1) * (dh + 1) + 1
        if H + 2 * pv < eh or W + 2 * ph < ew:
            continue
        OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
        C = int(g.choice([1, 3, 8, 17]))
        F = int(g.choice([1, 5, 16, 32, 33, 64, 96]))
        N = int(g.choice([2, 4, 8, 12, 16, 32, 64, 128]))
        if N * OH * OW * RH * RW * C * F > 4e8:
            continue
        act = [None, ("relu", 0.0), ("relu", 0.0), ("leaky_relu", 0.25), ("elu", 0.0), ("identity", 0.0)][int(g.integers(0, 6))]
        pools = [None]
        for prh in (1, 2, 3, 4):
            for prw in (1, 2, 4):
                if prh * prw > 1 and OH % prh == 0 and OW % prw == 0:
                    pools.append(("max", prh, prw, prh, prw))
        if OH >= 2 and OW >= 2:
            pools += [("mean", 2, 2, 2, 2), ("max", 2, 2, 1, 1)]
        pool = pools[int(g.integers(0, len(pools)))]
        if act is None and pool is None:
            continue
        out.append((N, H, W, C, F, dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh), act, pool))
    return out


SWEEP = _sweep_cases(120, 20250711)
SWEEP_MODES = {}


@pytest.mark.parametrize("index", range(len(SWEEP)))
def test_fused_sweep_exact(index):
    """Random fused groups on exactly representable data (see the module text): outputs, arg-max indices and every
    gradient equal the oracle's chain bit for bit, in whichever mode the group ran."""
    N, H, W, C, F, geom, act, pool = SWEEP[index]
    dtype = np.float32 if index % 3 else np.float64
    gen = hp.rng(4000 + index)
    x = _dyadic(gen, (N, H, W, C), dtype)
    w = _dyadic(gen, (geom["RH"] * geom["RW"] * C, F), dtype)
    b = _dyadic(gen, (1, F), dtype)
    if act is not None and act[0] == "elu":
        act = ("elu", 0.0)      # alpha 0: 0 * (exp(x) - 1) = 0 below zero, exact; the derivative there is y + alpha = 0
    fused, members, kdims = _build(dtype, N, H, W, C, F, conv=geom, act=act, pool=pool)
    chain = Chain(geom, act=act, pool=pool)
    x64, w64, b64 = (np.asarray(a, np.float64) for a in (x, w, b))
    ref = chain.forward(x64, w64, b64)
    g = _dyadic(gen, ref.shape, dtype)
    out, dx, mode = _run_fused(fused, members, x, w, b, g)
    SWEEP_MODES[mode] = SWEEP_MODES.get(mode, 0) + 1
    grads = chain.backward(x64, w64, np.asarray(g, np.float64))
    assert np.array_equal(out, ref), "output (%s)" % mode
    if pool is not None and pool[0] == "max":
        assert np.array_equal(members["pool"].max_indices(N), chain.inds), "arg-max indices (%s)" % mode
    wp, bp = members["conv"].get_params()
    assert np.array_equal(dx, grads["dx"]), "input gradient (%s)" % mode
    assert np.array_equal(wp.get_grad(), grads["dw"]), "weight gradient (%s)" % mode
    assert np.array_equal(bp.get_grad(), grads["db"].reshape(1, -1)), "bias gradient (%s)" % mode


def test_fused_sweep_met_every_mode():
    """Runs after the sweep: it must have exercised the epilogues, not only the member-by-member path."""
    if sum(SWEEP_MODES.values()) < len(SWEEP):
        pytest.skip("the sweep did not run in this session")
    assert SWEEP_MODES.get("pool", 0) >= 15 and SWEEP_MODES.get("act", 0) >= 15, SWEEP_MODES
