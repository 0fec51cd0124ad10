"""Copies between pageable host memory and the device: large ones are staged through pinned buffers by several
host threads (csrc/host_copy.hip); whatever the size, what comes back is what went in, byte for byte."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

MB = 1 << 20
# below the staging threshold, at it, one byte-group past a chunk, several chunks with a ragged tail, and more
# chunks than there are staging buffers
SIZES = [1, 1000, 4 * MB - 4, 4 * MB, 16 * MB + 12, 40 * MB + 68, 100 * MB + 4]


@pytest.mark.parametrize("nbytes", SIZES)
def test_round_trip_is_exact(nbytes):
    ch.init(0)
    n = nbytes // 4
    g = np.random.default_rng(nbytes)
    a = g.integers(0, 2 ** 32, size=n, dtype=np.uint32).view(np.float32).reshape((n, 1), order="F")
    t = ch.DeviceTensor.from_host(a)
    back = t.to_host()
    assert back.shape == a.shape
    assert np.array_equal(back.view(np.uint32), a.view(np.uint32))          # bit patterns, NaN payloads included
    t.free()


def test_upload_leaves_the_source_reusable_and_orders_with_kernels():
    """The source may be overwritten as soon as the upload returns, and a layer pass issued next sees the
    uploaded data (same stream)."""
    ch.init(0)
    dtype = np.float32
    shape = (64, 64, 64, 32)                    # 33.5 MB
    g = np.random.default_rng(7)
    x = np.asfortranarray(g.standard_normal(shape).astype(dtype))
    keep = x.copy(order="F")
    relu = ch.ActivationLayer(dtype, "relu", shape[1:])
    d = ch.DeviceTensor.from_host(x)
    x[...] = -1                                  # overwritten right after the upload
    y = ch.DeviceTensor(shape, dtype)
    relu.forward_into(d, y, True)
    assert np.array_equal(y.to_host(), np.maximum(keep, 0))


def test_layers_driven_from_two_threads():
    """Distinct layer objects may be driven from different threads at once (the reference's ParallelNeuralNetwork does,
    neural_network/ParallelNeuralNetwork.hpp:158-171); ctypes releases the interpreter lock during a call, so the
    calls of the two threads do overlap."""
    import threading
    ch.init(0)
    dtype = np.float32
    results = {}

    def work(tag, seed):
        g = np.random.default_rng(seed)
        x = np.asfortranarray(g.standard_normal((48, 20, 20, 8)).astype(dtype))      # 6 MB of output: staged copies too
        w = np.asfortranarray((0.2 * g.standard_normal((72, 40))).astype(dtype))
        layer = ch.ConvKernelLayer(dtype, (20, 20, 8), 40)
        layer.get_params()[0].set_values(w)
        outs = [layer.pass_forward(x, True) for _ in range(6)]
        results[tag] = (x, w, outs)

    threads = [threading.Thread(target=work, args=(i, 50 + i)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    from oracle import oracle
    for tag in range(2):
        x, w, outs = results[tag]
        ref, _ = oracle.conv_forward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.zeros((1, 40)), return_cache=True,
                                     RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0)
        for o in outs:
            assert np.array_equal(o, outs[0])
        err = np.max(np.abs(outs[0] - ref)) / np.sqrt(np.mean(ref ** 2))
        assert err < 1e-4
