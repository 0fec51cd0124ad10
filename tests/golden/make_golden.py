"""Writes tests/golden/layers_golden.npz: inputs and expected outputs of every hot-path layer.

The expected values do NOT come from the oracle: they are computed in float64 by independent
implementations available only in the development container (torch CPU autograd for convolution,
dense, batch norm, activations and pooling values; the definitional loops of tests/helpers.py for
the max-pool index encoding). The oracle must agree with them to 1e-10 before the file is written,
so the fixtures pin the oracle on machines that have neither torch nor the reference.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import helpers as hp  # noqa: E402
from oracle import oracle  # noqa: E402

OUT = os.path.join(HERE, "layers_golden.npz")
F64 = np.float64


def nchw(a):
    return torch.tensor(np.transpose(np.asarray(a, F64), (0, 3, 1, 2)).copy())


def nhwc(t):
    return np.asfortranarray(np.transpose(t.detach().numpy(), (0, 2, 3, 1)))


def agree(a, b, what):
    err = hp.rel_err(a, b)
    assert err < 1e-10, (what, err)


def conv_cases(store):
    # geometries of the reference's gradient tests (test/gradient_test.cpp:166-185) and the 3x3 p1 case
    for i, case in enumerate(hp.REFERENCE_CONV_CASES):
        H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
        g = hp.rng(7000 + i)
        N = 3
        x = hp.uniform(g, (N, H, W, C), -1, 1, F64)
        w = hp.uniform(g, (RH * RW * C, F), -1, 1, F64)
        b = hp.uniform(g, (1, F), -1, 1, F64)
        OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
        go = hp.uniform(g, (N, OH, OW, F), -1, 1, F64)
        xt = nchw(x).requires_grad_()
        # weight row k = rh + RH*(rw + RW*c)  (layer/kernel/ConvKernelLayer.hpp:128-142)
        wt = torch.tensor(np.transpose(w.reshape((RH, RW, C, F), order="F"), (3, 2, 0, 1)).copy(),
                          requires_grad=True)
        bt = torch.tensor(b.reshape(-1).copy(), requires_grad=True)
        out = torch.nn.functional.conv2d(xt, wt, bt, stride=(sv, sh), padding=(pv, ph),
                                         dilation=(dv + 1, dh + 1))
        out.backward(nchw(go))
        exp_out = nhwc(out)
        exp_dx = nhwc(xt.grad)
        exp_dw = np.asfortranarray(np.transpose(wt.grad.numpy(), (2, 3, 1, 0)).reshape((RH * RW * C, F),
                                                                                      order="F"))
        exp_db = bt.grad.numpy().reshape(1, F)
        geom = dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)
        o, cache = oracle.conv_forward(x, w, b, return_cache=True, **geom)
        dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **geom)
        for a, e, what in ((o, exp_out, "out"), (dx, exp_dx, "dx"), (dw, exp_dw, "dw"), (db, exp_db, "db")):
            agree(a, e, ("conv", i, what))
        p = "conv%d_" % i
        store.update({p + "case": np.array(case, np.int64), p + "x": x, p + "w": w, p + "b": b, p + "go": go,
                      p + "out": exp_out, p + "dx": exp_dx, p + "dw": exp_dw, p + "db": exp_db})


def dense_case(store):
    g = hp.rng(7100)
    N, dims, O = 5, (3, 2, 2), 7
    V = int(np.prod(dims))
    x = hp.uniform(g, (N,) + dims, -1, 1, F64)
    w = hp.uniform(g, (V, O), -1, 1, F64)
    b = hp.uniform(g, (1, O), -1, 1, F64)
    go = hp.uniform(g, (N, O), -1, 1, F64)
    xm = x.reshape((N, V), order="F")     # the reference's MatrixMap over the tensor (DenseKernelLayer.hpp:97)
    exp_out = xm @ w + b
    exp_dx = (go @ w.T).reshape(x.shape, order="F")
    exp_dw = xm.T @ go
    exp_db = go.sum(axis=0, keepdims=True)
    o = oracle.dense_forward(x, w, b)
    dx, dw, db = oracle.dense_backward(x, w, go)
    for a, e, what in ((o, exp_out, "out"), (dx, exp_dx, "dx"), (dw, exp_dw, "dw"), (db, exp_db, "db")):
        agree(a, e, ("dense", what))
    store.update({"dense_x": x, "dense_w": w, "dense_b": b, "dense_go": go, "dense_out": np.asfortranarray(exp_out),
                  "dense_dx": np.asfortranarray(exp_dx), "dense_dw": np.asfortranarray(exp_dw), "dense_db": exp_db})


def batchnorm_case(store):
    g = hp.rng(7200)
    N, H, W, C = 6, 4, 3, 5
    eps, decay = 1e-5, 0.1
    x1 = hp.normal(g, (N, H, W, C), F64, 2.0) + 0.5
    x2 = hp.normal(g, (N, H, W, C), F64, 1.0) - 0.25
    gamma = hp.uniform(g, (C,), 0.5, 1.5, F64).copy()
    beta = hp.uniform(g, (C,), -1, 1, F64).copy()
    go = hp.uniform(g, (N, H, W, C), -1, 1, F64)
    avg_mean = np.zeros(C)
    avg_inv_sd = np.zeros(C)
    exp = {}
    # two training passes (the first assigns the running statistics, the second averages them:
    # layer/BatchNormLayer.hpp:229-246), then one inference pass
    means, inv_sds = [], []
    for k, x in enumerate((x1, x2)):
        xt = nchw(x).requires_grad_()
        gt = torch.tensor(gamma.copy(), requires_grad=True)
        bt = torch.tensor(beta.copy(), requires_grad=True)
        yt = torch.nn.functional.batch_norm(xt, None, None, gt, bt, training=True, eps=eps)
        yt.backward(nchw(go))
        exp["y%d" % k], exp["dx%d" % k] = nhwc(yt), nhwc(xt.grad)
        exp["dgamma%d" % k], exp["dbeta%d" % k] = gt.grad.numpy(), bt.grad.numpy()
        flat = np.moveaxis(x, 3, 0).reshape(C, -1)
        means.append(flat.mean(axis=1))
        inv_sds.append(1.0 / np.sqrt(flat.var(axis=1) + eps))
    run_mean = (1 - decay) * means[0] + decay * means[1]
    run_inv_sd = (1 - decay) * inv_sds[0] + decay * inv_sds[1]
    exp["run_mean"], exp["run_inv_sd"] = run_mean, run_inv_sd
    exp["y_infer"] = np.asfortranarray((x1 - run_mean) * run_inv_sd * gamma + beta)
    for k, x in enumerate((x1, x2)):
        y, std, inv_sd = oracle.bn_forward(x, gamma, beta, avg_mean, avg_inv_sd, k > 0, True, True, decay, eps)
        dx, dg, db = oracle.bn_backward(go, gamma, std, inv_sd)
        for a, e, what in ((y, exp["y%d" % k], "y"), (dx, exp["dx%d" % k], "dx"), (dg, exp["dgamma%d" % k], "dg"),
                           (db, exp["dbeta%d" % k], "db")):
            agree(a, e, ("bn", k, what))
    agree(avg_mean, run_mean, "bn run mean")
    agree(avg_inv_sd, run_inv_sd, "bn run inv sd")
    y, _, _ = oracle.bn_forward(x1, gamma, beta, avg_mean, avg_inv_sd, True, False, True, decay, eps)
    agree(y, exp["y_infer"], "bn infer")
    store.update({"bn_x1": x1, "bn_x2": x2, "bn_gamma": gamma, "bn_beta": beta, "bn_go": go})
    store.update({"bn_" + k: v for k, v in exp.items()})


def activation_cases(store):
    g = hp.rng(7300)
    x = hp.uniform(g, (4, 5, 3, 2), -3, 3, F64)
    x[np.abs(x) < 1e-3] = 0.5          # keep clear of the kinks, where conventions differ
    go = hp.uniform(g, x.shape, -1, 1, F64)
    fn = torch.nn.functional
    acts = {
        "identity": (lambda t: t * 1.0, 0.0),
        "scaled": (lambda t: t * 1.7, 1.7),
        "sigmoid": (torch.sigmoid, 0.0),
        "tanh": (torch.tanh, 0.0),
        "softsign": (fn.softsign, 0.0),
        "softplus": (fn.softplus, 0.0),
        "relu": (torch.relu, 0.0),
        "leaky_relu": (lambda t: fn.leaky_relu(t, 0.1), 0.1),
        "elu": (lambda t: fn.elu(t, 0.8), 0.8),
        "swish": (lambda t: t * torch.sigmoid(1.3 * t), 1.3),
    }
    store.update({"act_x": x, "act_go": go})
    for name, (f, p) in acts.items():
        xt = torch.tensor(x.copy(), requires_grad=True)
        yt = f(xt)
        yt.backward(torch.tensor(go.copy()))
        y = oracle.act_forward(name, x, p)
        dx = oracle.act_backward(name, x, y, go, p)
        agree(y, yt.detach().numpy(), ("act", name, "y"))
        agree(dx, xt.grad.numpy(), ("act", name, "dx"))
        store.update({"act_%s_p" % name: np.array(p), "act_%s_y" % name: np.asfortranarray(yt.detach().numpy()),
                      "act_%s_dx" % name: np.asfortranarray(xt.grad.numpy())})
    # softmax over each sample's elements (layer/activation/SoftmaxActivationLayer.hpp:49-78); the
    # reference adds its epsilon to the denominator, which torch's softmax lacks
    xm = x.reshape((4, -1), order="F")
    e = np.exp(xm - xm.max(axis=1, keepdims=True))
    y_exp = e / (e.sum(axis=1, keepdims=True) + 1e-5)
    gm = go.reshape((4, -1), order="F")
    dx_exp = y_exp * (gm - (gm * y_exp).sum(axis=1, keepdims=True))
    y = oracle.softmax_forward(x, 1e-5)
    dx = oracle.softmax_backward(y, go)
    agree(y.reshape((4, -1), order="F"), y_exp, "softmax y")
    agree(dx.reshape((4, -1), order="F"), dx_exp, "softmax dx")
    store.update({"softmax_y": np.asfortranarray(y_exp.reshape(x.shape, order="F")),
                  "softmax_dx": np.asfortranarray(dx_exp.reshape(x.shape, order="F"))})
    # PReLU / PSwish: one parameter per element of a sample
    V = x.size // 4
    alpha = hp.uniform(g, (V,), 0.05, 0.4, F64).copy()
    beta = hp.uniform(g, (V,), 0.5, 1.5, F64).copy()
    for name, par, f in (("prelu", alpha, lambda t, a: torch.where(t > 0, t, a * t)),
                         ("pswish", beta, lambda t, b_: t * torch.sigmoid(b_ * t))):
        xt = torch.tensor(xm.copy(), requires_grad=True)
        pt = torch.tensor(par.copy(), requires_grad=True)
        yt = f(xt, pt)
        yt.backward(torch.tensor(gm.copy()))
        fwd = getattr(oracle, name + "_forward")
        bwd = getattr(oracle, name + "_backward")
        y = fwd(x, par)
        dx, dp = bwd(x, par, go)
        y_exp = yt.detach().numpy().reshape(x.shape, order="F")
        dx_exp = xt.grad.numpy().reshape(x.shape, order="F")
        agree(y, y_exp, (name, "y"))
        agree(dx, dx_exp, (name, "dx"))
        agree(dp, pt.grad.numpy(), (name, "dparam"))
        store.update({name + "_param": par, name + "_y": np.asfortranarray(y_exp),
                      name + "_dx": np.asfortranarray(dx_exp), name + "_dparam": pt.grad.numpy()})


def pool_cases(store):
    g = hp.rng(7400)
    # 2x2 stride 2 (the BASELINE networks) and the reference test's overlapping 3x2 stride (1,2) windows
    # (test/gradient_test.cpp:306,313)
    for i, (shape, RH, RW, sv, sh) in enumerate((((3, 8, 6, 4), 2, 2, 2, 2), ((2, 9, 8, 3), 3, 2, 1, 2))):
        x = hp.normal(g, shape, F64)
        if i == 0:
            x[0, 0:2, 0:2, 0] = 0.75       # a constant window: the first element wins
            x[1, 2, 2, 1] = x[1, 3, 3, 1] = 9.0   # two equal maxima: lower w (then lower h) wins
        OH, OW = (shape[1] - RH) // sv + 1, (shape[2] - RW) // sh + 1
        go = hp.uniform(g, (shape[0], OH, OW, shape[3]), -1, 1, F64)
        exp_max, exp_inds = hp.brute_maxpool(x, RH, RW, sv, sh)
        xt = nchw(x).requires_grad_()
        mt = torch.nn.functional.max_pool2d(xt, (RH, RW), (sv, sh))
        assert np.array_equal(nhwc(mt), exp_max)
        # scatter the gradient by the reference's index encoding k*RH + l (layer/pool/MaxPoolLayer.hpp:44-78)
        exp_max_dx = np.zeros(shape)
        N, C = shape[0], shape[3]
        for ow in range(OW):
            for oh in range(OH):
                for c in range(C):
                    for n in range(N):
                        bi = int(exp_inds[ow * OH + oh, c * N + n])
                        exp_max_dx[n, oh * sv + bi % RH, ow * sh + bi // RH, c] += go[n, oh, ow, c]
        xa = nchw(x).requires_grad_()
        at = torch.nn.functional.avg_pool2d(xa, (RH, RW), (sv, sh))
        at.backward(nchw(go))
        o, inds = oracle.maxpool_forward(x, RH, RW, sv, sh)
        assert np.array_equal(o, exp_max) and np.array_equal(inds, exp_inds)
        agree(oracle.maxpool_backward(shape, go, inds, RH, RW, sv, sh), exp_max_dx, "maxpool dx")
        agree(oracle.meanpool_forward(x, RH, RW, sv, sh), nhwc(at), "meanpool y")
        agree(oracle.meanpool_backward(shape, go, RH, RW, sv, sh), nhwc(xa.grad), "meanpool dx")
        p = "pool%d_" % i
        store.update({p + "geom": np.array((RH, RW, sv, sh), np.int64), p + "x": x, p + "go": go,
                      p + "max": exp_max, p + "inds": exp_inds, p + "max_dx": np.asfortranarray(exp_max_dx),
                      p + "mean": nhwc(at), p + "mean_dx": nhwc(xa.grad)})


def main():
    torch.manual_seed(0)
    store = {}
    conv_cases(store)
    dense_case(store)
    batchnorm_case(store)
    activation_cases(store)
    pool_cases(store)
    np.savez_compressed(OUT, **store)
    print("wrote %s: %d arrays, %d bytes" % (OUT, len(store), os.path.getsize(OUT)))


if __name__ == "__main__":
    main()
