"""A seeded sweep of convolution geometries (sizes, strides, dilations, paddings, batch sizes with and without 16-byte
alignment, filter counts around the tile widths) through forward, input gradient, weight and bias gradient, against
the CPU oracle in double precision. The fixed cases elsewhere pin known shapes; this one walks the launch policies
(tile shapes, split reductions, blocked tile rows, vector and scalar loads) with shapes nobody chose by hand."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")


def _cases(count, seed):
    g = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        RH, RW = int(g.integers(1, 5)), int(g.integers(1, 5))
        dv, dh = int(g.integers(0, 3)), int(g.integers(0, 3))
        sv, sh = int(g.integers(1, 4)), int(g.integers(1, 4))
        pv, ph = int(g.integers(0, RH)), int(g.integers(0, RW))
        H, W = int(g.integers(1, 24)), int(g.integers(1, 24))
        eh, ew = (RH - 1) * (dv + 1) + 1, (RW - 1) * (dh + 1) + 1          # extent of the dilated receptor
        if H + 2 * pv < eh or W + 2 * ph < ew:
            continue
        C = int(g.choice([1, 2, 3, 5, 8, 16, 21, 40]))
        F = int(g.choice([1, 3, 16, 31, 32, 33, 64, 65, 100, 128, 130]))
        N = int(g.choice([1, 2, 3, 4, 8, 12, 32, 33, 64, 96]))
        OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
        if N * OH * OW * RH * RW * C * F > 6e8:                            # keep the oracle to a fraction of a second
            continue
        out.append(((H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh), N))
    return out


def _tall_cases(count, seed):
    """Many output rows (thousands of 256-row tiles: whole rounds of the chip plus split left-over tiles, blocked
    tile rows when the batch is a multiple of 32), few channels so that the oracle stays fast."""
    g = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        N = int(g.choice([32, 64, 96, 128, 256]))
        H, W = int(g.integers(8, 41)), int(g.integers(8, 41))
        C = int(g.choice([1, 3, 4, 8]))
        F = int(g.choice([8, 16, 32, 48, 64, 128]))
        RH, RW = int(g.choice([1, 3])), int(g.choice([1, 3]))
        pv, ph = int(g.integers(0, RH)), int(g.integers(0, RW))
        sv, sh = int(g.choice([1, 1, 2])), int(g.choice([1, 1, 2]))
        OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, 0, 0)
        if N * OH * OW * RH * RW * C * F > 3e9:
            continue
        out.append(((H, W, C, F, RH, RW, pv, ph, sv, sh, 0, 0), N))
    return out


CASES = _cases(160, 20240611) + _tall_cases(32, 20240612)


@pytest.mark.parametrize("case,N", CASES, ids=["%dx%dx%d-f%d-r%dx%d-p%d%d-s%d%d-d%d%d-n%d" % (c + (n,)) for c, n in CASES])
def test_random_geometry(case, N):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    dtype = np.float32 if (H + W + C + F + N) % 3 else np.float64
    tol = 1e-4 if dtype == np.float32 else 1e-10
    g = hp.rng(1000 + H * 31 + W * 7 + C + F + N)
    x = hp.uniform(g, (N, H, W, C), -1, 1, dtype)
    w = hp.uniform(g, (RH * RW * C, F), -1, 1, dtype)
    b = hp.uniform(g, (1, F), -1, 1, dtype)
    OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    geom = dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **geom)
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, go64, **geom)
    assert out.shape == o_ref.shape
    assert hp.rel_err(out, o_ref) < tol, "forward"
    assert hp.rel_err(dx, dx_ref) < tol, "input gradient"
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol, "weight gradient"
    assert hp.rel_err(bp.get_grad(), db_ref) < tol, "bias gradient"


def _transconv_cases(count, seed):
    g = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        RH, RW = int(g.integers(1, 5)), int(g.integers(1, 5))
        dv, dh = int(g.integers(0, 2)), int(g.integers(0, 2))
        sv, sh = int(g.integers(1, 4)), int(g.integers(1, 4))
        pv, ph = int(g.integers(0, RH)), int(g.integers(0, RW))
        IH, IW = int(g.integers(1, 14)), int(g.integers(1, 14))
        OH, OW = oracle.transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh)
        if OH < 1 or OW < 1:
            continue
        C = int(g.choice([1, 2, 3, 8, 16, 33]))
        F = int(g.choice([1, 3, 16, 32, 40, 64]))
        N = int(g.choice([1, 3, 4, 8, 32, 33]))
        if N * OH * OW * RH * RW * C * F > 4e8:
            continue
        out.append(((IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh), N))
    return out


TRANS_CASES = _transconv_cases(64, 20240613)


@pytest.mark.parametrize("case,N", TRANS_CASES,
                         ids=["t%dx%dx%d-f%d-r%dx%d-p%d%d-s%d%d-d%d%d-n%d" % (c + (n,)) for c, n in TRANS_CASES])
def test_random_transposed_geometry(case, N):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    dtype = np.float32 if (IH + IW + C + F + N) % 3 else np.float64
    tol = 1e-4 if dtype == np.float32 else 1e-10
    geom = dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)
    g = hp.rng(2000 + IH * 31 + IW * 7 + C + F + N)
    OH, OW = oracle.transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh)
    x = hp.uniform(g, (N, IH, IW, C), -1, 1, dtype)
    w = hp.uniform(g, (C, RH * RW * F), -1, 1, dtype)
    b = hp.uniform(g, (1, OH * OW * F), -1, 1, dtype)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    layer = ch.TransConvKernelLayer(dtype, (IH, IW, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref = oracle.transconv_forward(x64, w64, b64, F, **geom)
    dx_ref, dw_ref, db_ref = oracle.transconv_backward(x64, w64, go64, **geom)
    assert out.shape == o_ref.shape
    assert hp.rel_err(out, o_ref) < tol, "forward"
    assert hp.rel_err(dx, dx_ref) < tol, "input gradient"
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol, "weight gradient"
    assert hp.rel_err(bp.get_grad(), db_ref) < tol, "bias gradient"


def _pool_cases(count, seed):
    g = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        RH, RW = int(g.integers(1, 5)), int(g.integers(1, 5))
        sv, sh = int(g.integers(1, 5)), int(g.integers(1, 5))
        H, W = int(g.integers(RH, RH + 20)), int(g.integers(RW, RW + 20))
        C = int(g.choice([1, 2, 3, 8, 17]))
        N = int(g.choice([1, 3, 4, 8, 32, 36, 64]))
        out.append((H, W, C, RH, RW, sv, sh, N))
    return out


POOL_SWEEP = _pool_cases(64, 20240614)


@pytest.mark.parametrize("H,W,C,RH,RW,sv,sh,N", POOL_SWEEP)
def test_random_pool_geometry(H, W, C, RH, RW, sv, sh, N):
    dtype = np.float32 if (H + W + C + N) % 2 else np.float64
    g = hp.rng(3000 + H * 31 + W * 7 + C + N)
    x = np.round(hp.normal(g, (N, H, W, C), dtype), 1)          # rounded: ties inside windows are common
    mx = ch.MaxPoolLayer(dtype, (H, W, C), RH, RW, sv, sh)
    out = mx.pass_forward(x, True)
    o_ref, i_ref = oracle.maxpool_forward(x, RH, RW, sv, sh)
    assert np.array_equal(out, o_ref)
    assert np.array_equal(mx.max_indices(N), i_ref)
    go = hp.normal(g, out.shape, dtype)
    assert np.array_equal(mx.pass_back(go), oracle.maxpool_backward(x.shape, go, i_ref, RH, RW, sv, sh))
    mn = ch.MeanPoolLayer(dtype, (H, W, C), RH, RW, sv, sh)
    tol = 1e-4 if dtype == np.float32 else 1e-10
    assert hp.rel_err(mn.pass_forward(x, True), oracle.meanpool_forward(np.asarray(x, np.float64), RH, RW, sv, sh)) < tol
    assert hp.rel_err(mn.pass_back(go), oracle.meanpool_backward(x.shape, np.asarray(go, np.float64), RH, RW, sv, sh)) < tol
