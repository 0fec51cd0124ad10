"""BASELINE configs 2, 3 and 5 end to end: the HIP layers driven by host-side counterparts of the
reference's callers (tests/harness.py) against the same orchestration on the CPU oracle.

Configs 2 and 3 are checked layer by layer at their real shapes and with their real data flow: every
oracle layer is fed exactly what the HIP layer was fed (forward activations and backward gradients
produced by the HIP network), so each comparison is a pure kernel comparison, max-pool argmax arrays
are compared bit for bit, and a rounding-level difference cannot flip a ReLU mask or an argmax
somewhere upstream. The optimizer step (reference formulas) is then applied to both."""
import numpy as np
import pytest

import harness as hn
import helpers as hp

pytestmark = pytest.mark.gpu
TOL = 1e-4          # fp32 max relative error (floor 0.1 RMS), the bound the benchmark definition states


def _sync_params(src_net, dst_net):
    for ps, pd in zip(src_net.params(), dst_net.params()):
        pd.set_values(np.asarray(ps.get_values(), np.float64))


def _layerwise_parity(hip, orc, x, obj, loss_grad):
    N = x.shape[0]
    acts, grads = [], []
    out = hn.train_step_gradients(hip, x, obj, loss_grad, acts, grads)
    # forward, teacher forced
    inp = np.asarray(x, np.float64)
    for i, lo in enumerate(orc.layers):
        ref = lo.pass_forward(inp, True)
        assert hp.rel_err(acts[i], ref) < TOL, "forward of layer %d" % i
        if hasattr(lo, "inds"):
            assert np.array_equal(hip.layers[i].max_indices(N), lo.inds), "argmax cache of layer %d" % i
        inp = np.asarray(acts[i], np.float64)
    # backward, teacher forced: grads[j] is what HIP layer L-1-j returned
    g = np.asarray(loss_grad(out, obj) / out.dtype.type(N), np.float64)
    L = len(orc.layers)
    for j in range(L):
        i = L - 1 - j
        ref = orc.layers[i].pass_back(np.asfortranarray(g))
        for k, (ph, po) in enumerate(zip(hip.layers[i].get_params(), orc.layers[i].get_params())):
            if not po.are_optimizable():
                continue
            got, want = np.asarray(ph.get_grad(), np.float64), po.get_grad()
            if want.shape[0] == 1 and g.ndim > 1:
                # A sum of the incoming gradient over everything but the last rank (bias, beta): in front
                # of a batch norm it is zero up to rounding, so the error is measured against the sum
                # of magnitudes of what was added up, not against the (cancelled) result.
                scale = np.abs(g).reshape((-1, g.shape[-1]), order="F").sum(axis=0)
                floor = np.maximum(np.maximum(np.abs(want.reshape(-1)), 1e-2 * scale), 1e-30)
                assert np.max(np.abs(got - want).reshape(-1) / floor) < TOL, "bias gradient of layer %d" % i
            else:
                assert hp.rel_err(got, want) < TOL, "gradient of parameter %d of layer %d" % (k, i)
        if i == 0:
            assert grads[j] is None and ref is None          # the input layer returns a null tensor
        else:
            label = "config 3 batchnorm dx" if type(orc.layers[i]).__name__ == "OracleBatchNorm" else None
            assert hp.rel_err(grads[j], ref, label=label) < TOL, "input gradient of layer %d" % i
            g = np.asarray(grads[j], np.float64)
    return out


def test_config2_mlp_sgd_step():
    """MLP 784 -> 512 -> 256 -> 10, ReLU, softmax cross-entropy, batch 256, one vanilla SGD step."""
    dt = np.float32
    gen = hp.rng(0xC0FFEE02)
    x = np.asfortranarray(gen.uniform(0, 1, (256, 784)).astype(dt))
    labels = gen.integers(0, 10, 256)
    obj = np.zeros((256, 10), dt, order="F")
    obj[np.arange(256), labels] = 1
    hip, orc = hn.build_mlp(hn.HipBackend(dt)), hn.build_mlp(hn.OracleBackend(np.float64))
    hn.init_kernel_weights(hip, 2, dt)
    _sync_params(hip, orc)
    _layerwise_parity(hip, orc, x, obj, hn.softmax_ce_grad)
    hn.vanilla_sgd_update(hip.params())
    hn.vanilla_sgd_update(orc.params())
    for ph, po in zip(hip.params(), orc.params()):
        assert hp.rel_err(ph.get_values(), po.get_values()) < TOL


def test_config3_convnet_adam_step():
    """conv32 -> ReLU -> pool -> conv64 -> BN -> ReLU -> pool -> dense10, batch 128, one Adam step."""
    dt = np.float32
    gen = hp.rng(0xC0FFEE03)
    x = np.asfortranarray(gen.standard_normal((128, 32, 32, 3)).astype(dt))
    labels = gen.integers(0, 10, 128)
    obj = np.zeros((128, 10, 1, 1), dt, order="F")
    obj[np.arange(128), labels, 0, 0] = 1
    hip, orc = hn.build_convnet(hn.HipBackend(dt)), hn.build_convnet(hn.OracleBackend(np.float64))
    hn.init_kernel_weights(hip, 3, dt)
    _sync_params(hip, orc)
    _layerwise_parity(hip, orc, x, obj, hn.softmax_ce_grad)
    # batch-norm running statistics after the first training pass (assigned, not blended)
    bn_h, bn_o = hip.layers[4].get_params(), orc.layers[4].get_params()
    assert hp.rel_err(bn_h[0].get_values(), bn_o[0].get_values()) < TOL
    assert hp.rel_err(bn_h[1].get_values(), bn_o[1].get_values()) < TOL
    ah, ao = hn.Adam(hip.params()), hn.Adam(orc.params())
    before = [np.array(p.get_values(), np.float64) for p in orc.params()]
    ah.update(hip.params())
    ao.update(orc.params())
    for ph, po, b in zip(hip.params(), orc.params(), before):
        if po.are_optimizable():
            # compare the update itself (new - old), which is what the step computes
            dh = np.asarray(ph.get_values(), np.float64) - b
            do = po.get_values() - b
            # an Adam step moves a weight by at most about lr = 1e-3: agree to a thousandth of that
            assert np.max(np.abs(dh - do)) < 1e-3 * 1e-3
            assert np.allclose(ph.get_values(), po.get_values(), rtol=TOL, atol=1e-6)


def test_config5_convlstm_bptt():
    """ConvLSTM, T=10, batch 32, 16x16x8 input, 32 hidden channels, MSE on the last hidden state, full BPTT.
    End to end against the float64 oracle network (all nonlinearities are smooth here)."""
    dt = np.float32
    gen = hp.rng(0xC0FFEE05)
    T, N = 10, 32
    x = np.asfortranarray(gen.standard_normal((N, T, 16, 16, 8)).astype(dt))
    target = np.asfortranarray(gen.standard_normal((N, 16, 16, 32)).astype(dt))
    hip, orc = hn.ConvLSTM(hn.HipBackend(dt), steps=T), hn.ConvLSTM(hn.OracleBackend(np.float64), steps=T)
    for (name, ph), (_, po) in zip(hip.kernel_params(), orc.kernel_params()):
        w = hn.he_normal(gen, ph[0].get_values().shape[0], 32, dt)
        ph[0].set_values(w)
        po[0].set_values(np.asarray(w, np.float64))
    out_h = hip.propagate(x)
    out_o = orc.propagate(np.asarray(x, np.float64))
    assert hp.rel_err(out_h, out_o) < TOL
    hip.backpropagate(np.asfortranarray(hn.squared_loss_grad(out_h, target) / dt(N)))
    orc.backpropagate(hn.squared_loss_grad(out_o, np.asarray(target, np.float64)) / N)
    for (name, ph), (_, po) in zip(hip.kernel_params(), orc.kernel_params()):
        assert hp.rel_err(ph[0].get_grad(), po[0].get_grad()) < TOL, name + " weights"
        assert hp.rel_err(ph[1].get_grad(), po[1].get_grad()) < TOL, name + " bias"
