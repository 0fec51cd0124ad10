"""State errors that must come back as status codes before any kernel is launched."""
import importlib

import numpy as np
import pytest

import helpers as hp

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")


def test_batchnorm_backward_after_an_inference_pass_of_another_batch_size():
    """A training pass at batch 8 fills the caches; an inference pass at batch 16 leaves them as they are; a backward
    pass at batch 16 would read past them (the reference asserts the row counts, BatchNormLayer.hpp:194)."""
    g = hp.rng(3)
    layer = ch.BatchNormLayer(np.float32, (4, 4, 3))
    layer.pass_forward(hp.normal(g, (8, 4, 4, 3), np.float32), True)
    layer.pass_forward(hp.normal(g, (16, 4, 4, 3), np.float32), False)
    with pytest.raises(ch.CattleHipError) as e:
        layer.pass_back(hp.normal(g, (16, 4, 4, 3), np.float32))
    assert e.value.code == 2
    # the matching batch size still works: the caches of the training pass are intact
    layer.pass_forward(hp.normal(g, (8, 4, 4, 3), np.float32), True)
    layer.pass_forward(hp.normal(g, (16, 4, 4, 3), np.float32), False)
    with pytest.raises(ch.CattleHipError):
        layer.pass_back(hp.normal(g, (8, 4, 4, 3), np.float32))      # the last forward pass had batch 16
    layer.pass_forward(hp.normal(g, (8, 4, 4, 3), np.float32), True)
    assert layer.pass_back(hp.normal(g, (8, 4, 4, 3), np.float32)).shape == (8, 4, 4, 3)


@pytest.mark.parametrize("make", [lambda: ch.ConvKernelLayer(np.float32, (6, 6, 2), 4),
                                  lambda: ch.ActivationLayer(np.float32, "relu", (6, 6, 2)),
                                  lambda: ch.TransConvKernelLayer(np.float32, (6, 6, 2), 4)])
def test_backward_after_the_borrowed_input_was_freed(make):
    """A layer borrows its device input until the backward pass; an input handed back to the pool in between may hold
    another tensor by then, so the backward pass is refused."""
    layer = make()
    x = ch.DeviceTensor.from_host(hp.normal(hp.rng(4), (8, 6, 6, 2), np.float32))
    out = ch.DeviceTensor((8,) + tuple(layer.get_output_dims()), np.float32)
    layer.forward_into(x, out, True)
    go = ch.DeviceTensor.from_host(hp.normal(hp.rng(5), out.shape, np.float32))
    dx = ch.DeviceTensor(x.shape, np.float32)
    x.free()
    with pytest.raises(ch.CattleHipError) as e:
        layer.backward_into(go, dx)
    assert e.value.code == 2
