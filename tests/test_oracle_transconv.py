"""Pins the oracle's transposed convolution (layer/kernel/TransConvKernelLayer.hpp:143-216) without the
reference being compilable: torch float64 conv_transpose2d with autograd as an independent implementation,
the adjoint identity with the (separately pinned) convolution, and the output-size formula on the geometries
of the reference's own gradient test (test/gradient_test.cpp:194-204)."""
import numpy as np
import pytest
import torch

import helpers as hp
from oracle import oracle

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}


def _inputs(case, N, dtype, seed):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    g = hp.rng(seed)
    OH, OW = oracle.transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh)
    x = hp.uniform(g, (N, IH, IW, C), -1, 1, dtype)
    w = hp.uniform(g, (C, RH * RW * F), -1, 1, dtype)
    b = hp.uniform(g, (1, OH * OW * F), -1, 1, dtype)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    return x, w, b, go


def _geom(case):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


def _torch_transconv(x, w, b, go, case):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    N = x.shape[0]
    xt = torch.tensor(np.transpose(np.asarray(x, np.float64), (0, 3, 1, 2)).copy(), requires_grad=True)
    # weight column rh + RH*(rw + RW*f) (TransConvKernelLayer.hpp:159-160) -> torch's (C_in, C_out, RH, RW)
    w4 = np.asarray(w, np.float64).reshape((C, RH, RW, F), order="F")
    wt = torch.tensor(np.transpose(w4, (0, 3, 1, 2)).copy(), requires_grad=True)
    out = torch.nn.functional.conv_transpose2d(xt, wt, None, stride=(sv, sh), padding=(pv, ph), dilation=(dv + 1, dh + 1))
    OH, OW = out.shape[2], out.shape[3]
    # one bias entry per output activation, in (oh, ow, f) column-major order (:172-173)
    bt = torch.tensor(np.transpose(np.asarray(b, np.float64).reshape((OH, OW, F), order="F"), (2, 0, 1)).copy(),
                      requires_grad=True)
    out = out + bt
    out.backward(torch.tensor(np.transpose(np.asarray(go, np.float64), (0, 3, 1, 2)).copy()))
    o = np.transpose(out.detach().numpy(), (0, 2, 3, 1))
    dx = np.transpose(xt.grad.numpy(), (0, 2, 3, 1))
    dw = np.transpose(wt.grad.numpy(), (0, 2, 3, 1)).reshape((C, RH * RW * F), order="F")
    db = np.transpose(bt.grad.numpy(), (1, 2, 0)).reshape((1, -1), order="F")
    return o, dx, dw, db


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", hp.REFERENCE_TRANSCONV_CASES)
def test_transconv_matches_torch(case, dtype):
    x, w, b, go = _inputs(case, 3, dtype, 300)
    o_t, dx_t, dw_t, db_t = _torch_transconv(x, w, b, go, case)
    out = oracle.transconv_forward(x, w, b, case[3], **_geom(case))
    dx, dw, db = oracle.transconv_backward(x, w, go, **_geom(case))
    tol = TOL[np.dtype(dtype)]
    assert out.shape == o_t.shape
    assert hp.rel_err(out, o_t) < tol and hp.rel_err(dx, dx_t) < tol
    assert hp.rel_err(dw, dw_t) < tol and hp.rel_err(db, db_t) < tol


def test_reference_test_geometries_give_the_documented_output_dims():
    # first layers of test/gradient_test.cpp:194-202 and the dims their second layers are built on
    assert oracle.transconv_out_dims(16, 1, 4, 1, 1, 0, 1, 1, 1, 0) == (20, 1)
    assert oracle.transconv_out_dims(4, 5, 5, 3, 1, 0, 1, 2, 0, 1) == (6, 13)
    assert oracle.transconv_out_dims(2, 3, 5, 3, 1, 0, 1, 2, 0, 1) == (4, 9)
    assert oracle.transconv_out_dims(4, 9, 2, 2, 1, 1, 1, 1, 0, 0) == (3, 8)


@pytest.mark.parametrize("case", hp.REFERENCE_TRANSCONV_CASES)
def test_transconv_is_the_adjoint_of_the_convolution(case):
    """<transconv(x; W), g> == <x, conv(g; W^T)> with zero biases: the transposed convolution is the input
    gradient of the convolution that maps its output back to its input."""
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    x, w, b, go = _inputs(case, 2, np.float64, 301)
    out = oracle.transconv_forward(x, w, np.zeros_like(b), F, **_geom(case))
    back = oracle.conv_forward(go, np.asfortranarray(w.T), np.zeros((1, C)), **_geom(case))
    assert back.shape == x.shape
    assert abs(np.vdot(out, go) - np.vdot(x, back)) < 1e-10 * max(1.0, abs(np.vdot(out, go)))


def test_transconv_gradients_accumulate_and_input_layer_skips():
    case = hp.REFERENCE_TRANSCONV_CASES[2]
    x, w, b, go = _inputs(case, 2, np.float64, 302)
    dx, dw, db = oracle.transconv_backward(x, w, go, **_geom(case))
    dx2, dw2, db2 = oracle.transconv_backward(x, w, go, wgrad=dw.copy(order="F"), bgrad=db.copy(order="F"), input_layer=True,
                                              **_geom(case))
    assert dx2 is None
    assert hp.rel_err(dw2, 2 * dw) < 1e-12 and hp.rel_err(db2, 2 * db) < 1e-12
