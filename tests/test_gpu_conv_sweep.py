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
