"""The entry point that allocates nothing (cattle_hip_conv_forward_noalloc) against the layer entry point it is a
variant of (cattle_hip_layer_forward on a convolution layer): same kernels, same launch plan, so the outputs must
agree bit for bit. Two calls in a row share the library's fixed scratch array, the second with a smaller input."""
import importlib

import numpy as np
import pytest

import helpers as hp

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")


def _both(dtype, N, H, W, C, F, seed, geom=(3, 3, 1, 1, 1, 1, 0, 0), bias=True):
    RH, RW, pv, ph, sv, sh, dv, dh = geom
    g = hp.rng(seed)
    x = hp.normal(g, (N, H, W, C), dtype)
    w = hp.normal(g, (RH * RW * C, F), dtype, std=0.2)
    b = hp.normal(g, (1, F), dtype) if bias else np.zeros((1, F), dtype, order="F")
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
    layer.get_params()[0].set_values(w)
    layer.get_params()[1].set_values(b)
    xd, wd, bd = (ch.DeviceTensor.from_host(a) for a in (x, w, b))
    want = layer.pass_forward(xd, True).to_host()
    out = ch.DeviceTensor(want.shape, dtype)
    ch.conv_forward_noalloc(xd, wd, bd if bias else None, out, RH, RW, pv, ph, sv, sh, dv, dh)
    return out.to_host(), want


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_two_calls_in_a_row_match_the_layer_entry_point(dtype):
    # a reduction cut into parts (few rows, K = 288): the partial sums go through the static scratch array
    got, want = _both(dtype, 32, 16, 16, 32, 128, seed=5)
    assert np.array_equal(got, want)
    # a smaller input right after it: stale partial sums and stale prepared weights of the first call are still there
    got, want = _both(dtype, 16, 8, 8, 16, 24, seed=6, geom=(3, 2, 1, 0, 1, 2, 0, 0))
    assert np.array_equal(got, want)
    # whole tiles plus left-over tiles whose reduction is cut (a tall problem), without bias
    got, want = _both(dtype, 64, 28, 28, 32, 64, seed=7, bias=False)
    assert np.array_equal(got, want)


def test_too_large_for_the_scratch_array_is_refused_and_nothing_is_allocated():
    free0, _ = ch.memory_info()
    assert ch.static_scratch_bytes() == 72 << 20
    # weights alone exceed the array: 9 * 4096 rows x 4096 columns of fp64 = 1.2 GB (no kernel is launched)
    N, H, W, C, F = 1, 4, 4, 4096, 4096
    x = ch.DeviceTensor((N, H, W, C), np.float64)
    w = ch.DeviceTensor((9 * C, F), np.float64)
    out = ch.DeviceTensor((N, H, W, F), np.float64)
    free1, _ = ch.memory_info()
    with pytest.raises(ch.CattleHipError) as e:
        ch.conv_forward_noalloc(x, w, None, out)
    assert e.value.code == 1 and "static scratch buffer" in str(e.value)
    # a problem that fits: the device's free memory does not move across the call
    x2 = ch.DeviceTensor.from_host(hp.normal(hp.rng(1), (32, 16, 16, 32), np.float32))
    w2 = ch.DeviceTensor.from_host(hp.normal(hp.rng(2), (288, 128), np.float32))
    o2 = ch.DeviceTensor((32, 16, 16, 128), np.float32)
    ch.conv_forward_noalloc(x2, w2, None, o2)
    ch.synchronize()
    before, _ = ch.memory_info()
    for _ in range(3):
        ch.conv_forward_noalloc(x2, w2, None, o2)
    after, _ = ch.memory_info()
    assert after == before
