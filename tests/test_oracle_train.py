"""Pins the oracle's loss functions and optimizer updates (the two ends of a training step around the
layer stack) without the reference being compilable: torch float64 as an independent implementation
where the formulas coincide, closed forms, central differences, and the time-step slicing property
of the sequential losses. The reference's own tests hold no known answers for these either."""
import numpy as np
import pytest
import torch

import helpers as hp
from oracle import oracle

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]


def _one_hot(gen, N, V, dtype):
    y = np.zeros((N, V), dtype=dtype, order="F")
    y[np.arange(N), gen.integers(0, V, N)] = 1
    return y


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_cross_entropy_against_torch(dtype):
    g = hp.rng(901)
    N, V = 9, 10
    out = hp.normal(g, (N, V), dtype, 3.0)
    obj = _one_hot(g, N, V, dtype)
    ot = torch.tensor(np.asarray(out, np.float64), requires_grad=True)
    yt = torch.tensor(np.asarray(obj, np.float64))
    lt = torch.nn.functional.cross_entropy(ot, yt, reduction="none")
    lt.sum().backward()
    # epsilon 0: the reference's formula is then exactly -sum y log softmax, and its gradient
    # softmax - y is the true derivative because each row of y sums to one
    assert hp.rel_err(oracle.loss_function("softmax_cross_entropy", out, obj, eps=0.0), lt.detach().numpy()) < TOL[np.dtype(dtype)]
    assert hp.rel_err(oracle.loss_d_function("softmax_cross_entropy", out, obj, eps=0.0), ot.grad.numpy()) < TOL[np.dtype(dtype)]
    # the scale multiplies the gradient (the optimizer's division by the batch size)
    assert hp.rel_err(oracle.loss_d_function("softmax_cross_entropy", out, obj, eps=0.0, scale=1.0 / 128),
                      ot.grad.numpy() / 128) < TOL[np.dtype(dtype)]


def test_softmax_cross_entropy_epsilon_and_soft_targets():
    """With the epsilon in the denominator and arbitrary targets: p = e / (sum e + eps), L = -sum log(p) y,
    grad = p - y (not the derivative of L unless the targets sum to one: the reference's choice)."""
    g = hp.rng(902)
    N, V, eps = 6, 7, 1e-2          # a large epsilon so that a misplaced one shows
    out = hp.normal(g, (N, V), np.float64, 2.0)
    obj = hp.uniform(g, (N, V), 0, 1, np.float64)
    e = np.exp(out - out.max(axis=1, keepdims=True))
    p = e / (e.sum(axis=1, keepdims=True) + eps)
    assert hp.rel_err(oracle.loss_function("softmax_cross_entropy", out, obj, eps=eps), -(np.log(p) * obj).sum(axis=1)) < 1e-12
    assert hp.rel_err(oracle.loss_d_function("softmax_cross_entropy", out, obj, eps=eps), p - obj) < 1e-12
    # shifting a row by a constant changes nothing (the max subtraction)
    shifted = out + np.arange(N).reshape(N, 1) * 10.0
    assert hp.rel_err(oracle.loss_function("softmax_cross_entropy", shifted, obj, eps=eps),
                      oracle.loss_function("softmax_cross_entropy", out, obj, eps=eps)) < 1e-12


@pytest.mark.parametrize("dtype", DTYPES)
def test_squared_loss_against_torch(dtype):
    g = hp.rng(903)
    N, dims = 5, (4, 3, 2)
    out = hp.normal(g, (N,) + dims, dtype)
    obj = hp.normal(g, (N,) + dims, dtype)
    ot = torch.tensor(np.asarray(out, np.float64), requires_grad=True)
    lt = torch.nn.functional.mse_loss(ot, torch.tensor(np.asarray(obj, np.float64)), reduction="none").reshape(N, -1).sum(dim=1)
    lt.sum().backward()
    assert hp.rel_err(oracle.loss_function("squared", out, obj), lt.detach().numpy()) < TOL[np.dtype(dtype)]
    assert hp.rel_err(oracle.loss_d_function("squared", out, obj), ot.grad.numpy()) < TOL[np.dtype(dtype)]


@pytest.mark.parametrize("kind", ["squared", "softmax_cross_entropy"])
def test_loss_gradient_is_the_derivative(kind):
    """Central differences of sum(function) against d_function (targets sum to one, tiny epsilon)."""
    g = hp.rng(904)
    N, V = 4, 6
    out = hp.normal(g, (N, V), np.float64)
    obj = _one_hot(g, N, V, np.float64) if kind != "squared" else hp.normal(g, (N, V), np.float64)
    grad = oracle.loss_d_function(kind, out, obj, eps=1e-14)
    h = 1e-6
    for n in range(N):
        for j in range(V):
            up, dn = out.copy(order="F"), out.copy(order="F")
            up[n, j] += h
            dn[n, j] -= h
            num = (oracle.loss_function(kind, up, obj, eps=1e-14).sum() - oracle.loss_function(kind, dn, obj, eps=1e-14).sum()) / (2 * h)
            assert abs(num - grad[n, j]) < 1e-7


def _torch_loss(kind, o, y):
    """Independent float64 implementations (torch's own loss routines where it has one) of the losses at
    epsilon 0, as differentiable per-sample values; o, y are (N, V) torch tensors."""
    F = torch.nn.functional
    V = o.shape[1]
    if kind == "absolute":
        return F.l1_loss(o, y, reduction="none").sum(dim=1)
    if kind == "binary_cross_entropy":
        return F.binary_cross_entropy(o, y, reduction="none").sum(dim=1)
    if kind == "cross_entropy":            # one-hot objectives: the negative log likelihood of the class
        return F.nll_loss(torch.log(o), y.argmax(dim=1), reduction="none")
    if kind == "kullback_leibler":         # -sum y ln(o / y) = KL(y || o)
        return F.kl_div(torch.log(o), y, reduction="none").sum(dim=1)
    if kind in ("hinge", "squared_hinge"):  # torch averages over the classes, the reference sums
        return F.multi_margin_loss(o, y.argmax(dim=1), p=2 if kind == "squared_hinge" else 1, margin=1.0, reduction="none") * V
    if kind in ("multi_label_hinge", "squared_multi_label_hinge"):
        m = torch.clamp(1 - y * o, min=0)
        return (m * m if kind == "squared_multi_label_hinge" else m).sum(dim=1)
    if kind == "multi_label_log":          # the reference's value is the log likelihood itself, not its negative
        return -F.binary_cross_entropy(o, y, reduction="none").sum(dim=1)
    raise KeyError(kind)


@pytest.mark.parametrize("kind", hp.ALL_LOSSES[2:])
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_other_losses_against_torch(kind, dtype):
    g = hp.rng(910)
    N, V = 7, (1 if kind == "binary_cross_entropy" else 6)
    src = "hinge" if kind == "cross_entropy" else kind          # one-hot objectives for the nll comparison
    out, obj = hp.loss_inputs(g, src, N, (V,), dtype)
    if kind == "cross_entropy":
        out = hp.loss_inputs(g, kind, N, (V,), dtype)[0]
    ot = torch.tensor(np.asarray(out, np.float64), requires_grad=True)
    lt = _torch_loss(kind, ot, torch.tensor(np.asarray(obj, np.float64)))
    lt.sum().backward()
    tol = TOL[np.dtype(dtype)]
    assert hp.rel_err(oracle.loss_function(kind, out, obj, eps=0.0), lt.detach().numpy()) < tol
    assert hp.rel_err(oracle.loss_d_function(kind, out, obj, eps=0.0), ot.grad.numpy()) < tol
    assert hp.rel_err(oracle.loss_d_function(kind, out, obj, eps=0.0, scale=0.25), ot.grad.numpy() / 4) < tol
    # NegatedLoss (loss/NegatedLoss.hpp:41-46)
    assert np.array_equal(oracle.loss_function(kind, out, obj, eps=0.0, negated=True), -oracle.loss_function(kind, out, obj, eps=0.0))
    assert np.array_equal(oracle.loss_d_function(kind, out, obj, eps=0.0, scale=0.25, negated=True),
                          -oracle.loss_d_function(kind, out, obj, eps=0.0, scale=0.25))


def test_losses_hand_worked_rows():
    """Rows small enough to work by hand, with epsilons large enough that a misplaced one shows, and the hinge
    losses at their thresholds."""
    f64 = np.float64
    col = lambda *v: np.asfortranarray(np.array(v, f64).reshape(1, -1))
    ln = np.log
    # binary cross entropy, one value per sample: -(y ln(o + e) + (1 - y) ln((1 + e) - o)),  e = 0.25
    o, y = np.asfortranarray(np.array([[0.25], [0.25]], f64)), np.asfortranarray(np.array([[1.0], [0.0]], f64))
    assert np.allclose(oracle.loss_function("binary_cross_entropy", o, y, eps=0.25), [ln(2.0), 0.0], atol=1e-15)
    assert np.allclose(oracle.loss_d_function("binary_cross_entropy", o, y, eps=0.25)[:, 0], [-2.0, 1.0], atol=1e-15)
    with pytest.raises(RuntimeError):
        oracle.loss_function("binary_cross_entropy", col(0.2, 0.3), col(1, 0))         # more than one value per sample
    # cross entropy: -ln(o + e) y ; gradient -y / (o + e)
    assert np.allclose(oracle.loss_function("cross_entropy", col(0.25, 0.5), col(1, 0), eps=0.25), [ln(2.0)], atol=1e-15)
    assert np.allclose(oracle.loss_d_function("cross_entropy", col(0.25, 0.5), col(1, 0.5), eps=0.25), [[-2.0, -2.0 / 3]], atol=1e-15)
    # Kullback-Leibler: -ln(o / (y + e) + e) y ; the reference's gradient is the cross entropy's, -y / (o + e)
    assert np.allclose(oracle.loss_function("kullback_leibler", col(1.0, 3.0), col(0.5, 0.0), eps=0.5), [-0.5 * ln(1.5)], atol=1e-15)
    assert np.allclose(oracle.loss_d_function("kullback_leibler", col(1.0, 3.0), col(0.5, 0.0), eps=0.5), [[-1.0 / 3, 0.0]], atol=1e-15)
    # multi-label log: sum y ln(o + e) + (1 - y) ln(1 + e - o); gradient (y - o) / (o (1 - o)), where an output of
    # exactly 0 becomes e in the numerator only, so the quotient is infinite
    assert np.allclose(oracle.loss_function("multi_label_log", col(0.25, 0.75), col(1, 0), eps=0.25), [2 * ln(0.5)], atol=1e-15)
    assert np.allclose(oracle.loss_d_function("multi_label_log", col(0.25, 0.5), col(1, 0), eps=0.25), [[4.0, -2.0]], atol=1e-15)
    with np.errstate(all="ignore"):
        inf = oracle.loss_d_function("multi_label_log", col(0.0, 0.0), col(1, 0), eps=0.25)
    assert inf[0, 0] == np.inf and inf[0, 1] == -np.inf
    # absolute: a zero difference has gradient +1 (loss/AbsoluteLoss.hpp:34)
    assert np.array_equal(oracle.loss_d_function("absolute", col(1.0, 2.0, 0.5), col(1.0, 3.0, 0.25)), [[1.0, -1.0, 1.0]])
    assert np.array_equal(oracle.loss_function("absolute", col(1.0, 2.0, 0.5), col(1.0, 3.0, 0.25)), [1.25])
    # hinge, class 0 with score 2: margins of the others are 0 (no loss, no gradient), 0.5, and half a machine
    # epsilon (counted by the loss, not "decidedly greater" than 0 for the gradient: core/NumericUtils.hpp:62-65)
    tiny = np.finfo(f64).eps / 2
    o, y = col(2.0, 1.0, 1.5, 1.0 + tiny * 2), col(1, 0, 0, 0)       # 1 + 2 tiny is the next double after 1
    assert o[0, 3] - 2.0 + 1 == tiny * 2
    assert np.allclose(oracle.loss_function("hinge", o, y), [0.5 + 2 * tiny], atol=1e-18)
    assert np.array_equal(oracle.loss_d_function("hinge", o, y), [[-1.0, 0.0, 1.0, 0.0]])
    assert np.allclose(oracle.loss_function("squared_hinge", o, y), [0.25], atol=1e-18)
    assert np.array_equal(oracle.loss_d_function("squared_hinge", o, y), [[-1.0, 0.0, 1.0, 0.0]])
    # the class is the LAST element that equals one (loss/HingeLoss.hpp:44-47); a row without a one is refused
    assert np.array_equal(oracle.loss_d_function("hinge", col(0.0, 0.0, 5.0), col(0, 1, 0)), [[1.0, -2.0, 1.0]])
    with pytest.raises(RuntimeError):
        oracle.loss_function("hinge", col(0.0, 1.0), col(0, 0))
    # multi-label hinge: max(0, 1 - y o); gradient -y, squared 2 o - 2 y, inside the margin only
    o, y = col(0.5, -2.0, 1.0, -0.25), col(1, -1, 1, 1)
    assert np.array_equal(oracle.loss_function("multi_label_hinge", o, y), [0.5 + 0 + 0 + 1.25])
    assert np.array_equal(oracle.loss_d_function("multi_label_hinge", o, y), [[-1.0, 0.0, 0.0, -1.0]])
    assert np.array_equal(oracle.loss_function("squared_multi_label_hinge", o, y), [0.25 + 1.5625])
    assert np.array_equal(oracle.loss_d_function("squared_multi_label_hinge", o, y), [[-1.0, 0.0, 0.0, -2.5]])


@pytest.mark.parametrize("kind", hp.ALL_LOSSES[2:])
def test_the_other_losses_gradients_are_the_derivatives(kind):
    """Central differences, as in the reference's own loss tests (test/gradient_test.cpp:819-1100), with an epsilon
    small enough for the reference's simplified gradients to be the derivatives."""
    g = hp.rng(911)
    N, V = 3, (1 if kind == "binary_cross_entropy" else 5)
    out, obj = hp.loss_inputs(g, kind, N, (V,), np.float64)
    grad = oracle.loss_d_function(kind, out, obj, eps=1e-14)
    h = 1e-6
    for n in range(N):
        for j in range(V):
            up, dn = out.copy(order="F"), out.copy(order="F")
            up[n, j] += h
            dn[n, j] -= h
            num = (oracle.loss_function(kind, up, obj, eps=1e-14).sum() - oracle.loss_function(kind, dn, obj, eps=1e-14).sum()) / (2 * h)
            assert abs(num - grad[n, j]) < 1e-6 * max(1.0, abs(grad[n, j]))


@pytest.mark.parametrize("kind", hp.ALL_LOSSES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_sequential_losses_are_per_time_step(kind, dtype):
    """loss/UniversalLoss.hpp:99-125: every time step is sliced out and handled as a non-sequential batch;
    losses add up over the steps, gradients are written back into the step's slice."""
    g = hp.rng(905)
    N, Ts, dims = 5, 4, ((1, 1) if kind == "binary_cross_entropy" else (3, 2))
    out, obj = hp.loss_inputs(g, kind, N, dims, dtype, steps=Ts)
    total = oracle.loss_function(kind, out, obj, sequential=True)
    grad = oracle.loss_d_function(kind, out, obj, scale=0.5, sequential=True)
    acc = np.zeros(N)
    for t in range(Ts):
        o_t, y_t = np.asfortranarray(out[:, t]), np.asfortranarray(obj[:, t])
        acc += oracle.loss_function(kind, o_t, y_t)
        assert hp.rel_err(grad[:, t], oracle.loss_d_function(kind, o_t, y_t, scale=0.5)) < TOL[np.dtype(dtype)]
    assert hp.rel_err(total, acc) < TOL[np.dtype(dtype)]


def test_regularization_by_hand_and_by_differences():
    """parameter_regularization/*.hpp: L1 = lambda sum |v| with gradient +-lambda (+lambda at zero), L2 = lambda / 2 sum v^2
    with gradient lambda v, the elastic net their sum."""
    v = np.asfortranarray(np.array([[1.0, -2.0], [0.0, 0.5]]))
    pen, grad = oracle.regularization(v, l1=0.1)
    assert abs(pen - 0.35) < 1e-15 and np.array_equal(grad, [[0.1, -0.1], [0.1, 0.1]])
    pen, grad = oracle.regularization(v, l2=0.2)
    assert abs(pen - 0.1 * 5.25) < 1e-15 and np.allclose(grad, [[0.2, -0.4], [0.0, 0.1]], atol=1e-16)
    pen, grad = oracle.regularization(v, l1=0.1, l2=0.2)
    assert abs(pen - 0.875) < 1e-15 and np.allclose(grad, [[0.3, -0.5], [0.1, 0.2]], atol=1e-16)
    pen, grad = oracle.regularization(v)
    assert pen == 0 and np.all(grad == 0)
    g = hp.rng(920)
    w = hp.normal(g, (5, 4), np.float64)
    _, grad = oracle.regularization(w, l1=0.03, l2=0.7)
    h = 1e-6
    for idx in [(0, 0), (2, 3), (4, 1)]:
        up, dn = w.copy(order="F"), w.copy(order="F")
        up[idx] += h
        dn[idx] -= h
        num = (oracle.regularization(up, l1=0.03, l2=0.7)[0] - oracle.regularization(dn, l1=0.03, l2=0.7)[0]) / (2 * h)
        assert abs(num - grad[idx]) < 1e-8


def test_parameter_constraints_by_hand():
    """StandardParameters.hpp:150-182 on a 3-4-5 matrix: the clip, the "L1" constraint that measures the Euclidean norm, the
    "L2" constraint that compares the squared norm with its limit and scales by their ratio (so that a matrix over the limit
    ends up with the squared norm limit^2 / old squared norm, not with the limit), their order, and limits that are off."""
    m = np.asfortranarray(np.array([[3.0, -4.0]]))
    assert np.array_equal(oracle.constrain(m), m)
    assert np.array_equal(oracle.constrain(m, clip=3.5), [[3.0, -3.5]])
    assert np.array_equal(oracle.constrain(m, clip=1e-17), m)                        # not decidedly greater than zero: off
    assert np.allclose(oracle.constrain(m, max_l1_norm=2.5), [[1.5, -2.0]], rtol=1e-15)   # norm() = 5: halved
    assert np.array_equal(oracle.constrain(m, max_l1_norm=5.0), m)                   # not over the limit
    assert np.array_equal(oracle.constrain(m, max_l1_norm=6.9), m)                   # an L1 norm of 7 would be over: not what is measured
    out = oracle.constrain(m, max_l2_norm=5.0)                                       # squaredNorm() = 25 > 5: scaled by 5 / 25
    assert np.allclose(out, [[0.6, -0.8]], rtol=1e-15) and abs(np.sum(out * out) - 1.0) < 1e-15
    assert np.array_equal(oracle.constrain(m, max_l2_norm=25.0), m)
    # order: clip to [-3.5, 3.5] -> (3, -3.5), norm sqrt(21.25) > 2 -> scaled to norm 2 (squared norm 4) -> 4 > 1 -> scaled by 1 / 4
    out = oracle.constrain(m, clip=3.5, max_l1_norm=2.0, max_l2_norm=1.0)
    want = np.array([[3.0, -3.5]]) * (2.0 / np.sqrt(21.25)) * 0.25
    assert np.allclose(out, want, rtol=1e-14)
    out32 = oracle.constrain(m.astype(np.float32), clip=3.5, max_l1_norm=2.0, max_l2_norm=1.0)
    assert out32.dtype == np.float32 and np.allclose(out32, want, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_l2_regularized_sgd_is_torch_weight_decay(dtype):
    """SGDOptimizer::_train regularizes, then updates (optimizer/SGDOptimizer.hpp:59-64): with L2 regularization and
    vanilla SGD that is torch's SGD with weight_decay = lambda."""
    g = hp.rng(921)
    w0, lam, lr = hp.normal(g, (6, 4), dtype), 0.05, 0.1
    wt = torch.tensor(np.asarray(w0, np.float64), requires_grad=True)
    opt = torch.optim.SGD([wt], lr=lr, weight_decay=lam)
    w = w0
    for _ in range(3):
        grad = hp.normal(g, (6, 4), dtype)
        wt.grad = torch.tensor(np.asarray(grad, np.float64))
        opt.step()
        _, reg = oracle.regularization(w, l2=lam)
        w = oracle.sgd_update(w, grad + reg, lr)
    assert hp.rel_err(w, wt.detach().numpy()) < TOL[np.dtype(dtype)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_sgd_update(dtype):
    g = hp.rng(906)
    w = hp.normal(g, (7, 5), dtype)
    dw = hp.normal(g, (7, 5), dtype)
    new = oracle.sgd_update(w, dw, lr=0.05)
    assert hp.rel_err(new, np.asarray(w, np.float64) - 0.05 * np.asarray(dw, np.float64)) < TOL[np.dtype(dtype)]
    assert np.array_equal(oracle.sgd_update(w, np.zeros_like(dw), lr=0.05), w)


def test_adam_first_step_is_a_signed_step():
    """From zero moving averages, step 0, epsilon -> 0: m = d1 g, v = d2 g^2, both corrections undo the
    decay factors, so the update is lr * g / |g| whatever the decay rates are."""
    g = hp.rng(907)
    w = hp.normal(g, (6, 4), np.float64)
    dw = hp.uniform(g, (6, 4), 0.5, 2.0, np.float64) * np.where(g.random((6, 4)) < 0.5, -1, 1)
    z = np.zeros_like(w)
    for d1, d2 in ((0.1, 0.001), (0.3, 0.05)):
        new, m, v = oracle.adam_update(w, dw, z, z, 0, lr=0.01, l1_decay=d1, l2_decay=d2, eps=1e-30)
        assert np.max(np.abs(new - (w - 0.01 * np.sign(dw)))) < 1e-12
        assert hp.rel_err(m, d1 * dw) < 1e-12 and hp.rel_err(v, d2 * dw * dw) < 1e-12


def test_adam_matches_torch_in_the_small_epsilon_limit():
    """torch's Adam divides by sqrt(v_hat) + eps and corrects by 1 - beta^t; the reference divides by
    sqrt(v_hat + eps) and corrects by 1 - beta^t + eps. For eps -> 0 they are the same recurrence with
    beta = 1 - decay, so several steps with changing gradients must agree."""
    g = hp.rng(908)
    w0 = hp.normal(g, (5, 3), np.float64)
    grads = [hp.uniform(g, (5, 3), 0.5, 2.0, np.float64) * np.where(g.random((5, 3)) < 0.5, -1, 1) for _ in range(6)]
    d1, d2, lr = 0.1, 0.01, 0.02
    pt = torch.tensor(w0.copy(), requires_grad=True)
    opt = torch.optim.Adam([pt], lr=lr, betas=(1 - d1, 1 - d2), eps=1e-30)
    w, m, v = w0, np.zeros_like(w0), np.zeros_like(w0)
    for t, dw in enumerate(grads):
        pt.grad = torch.tensor(dw.copy())
        opt.step()
        w, m, v = oracle.adam_update(w, dw, m, v, t, lr=lr, l1_decay=d1, l2_decay=d2, eps=1e-30)
        assert np.max(np.abs(w - pt.detach().numpy())) < 1e-12, t


@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_reference_formula_with_default_epsilon(dtype):
    """The reference's exact placement of epsilon (optimizer/AdamOptimizer.hpp:67-81), evaluated
    independently in vectorised float64 over three steps."""
    g = hp.rng(909)
    w = hp.normal(g, (8, 3), dtype)
    lr, d1, d2, eps = 1e-3, 1e-1, 1e-3, 1e-5
    w64, m64, v64 = np.asarray(w, np.float64), np.zeros((8, 3)), np.zeros((8, 3))
    m, v = np.zeros_like(w), np.zeros_like(w)
    for t in range(3):
        dw = hp.normal(g, (8, 3), dtype)
        w, m, v = oracle.adam_update(w, dw, m, v, t, lr, d1, d2, eps)
        c1 = 1.0 / (1 - (1 - d1) ** (t + 1) + eps)
        c2 = 1.0 / (1 - (1 - d2) ** (t + 1) + eps)
        m64 = (1 - d1) * m64 + d1 * dw
        v64 = (1 - d2) * v64 + d2 * np.square(np.asarray(dw, np.float64))
        w64 = w64 - lr * c1 * m64 / np.sqrt(c2 * v64 + eps)
        assert hp.rel_err(w, w64) < TOL[np.dtype(dtype)]
        assert hp.rel_err(m, m64) < TOL[np.dtype(dtype)] and hp.rel_err(v, v64) < TOL[np.dtype(dtype)]


# ---------------------------------------------------------------------------------------------------------
# The other optimizers (optimizer/*.hpp). torch's implementations are independent code; where the
# reference's recurrence is the same one (possibly after mapping the hyper-parameters) several steps with
# changing gradients must agree. Nadam and AMSGrad differ from torch's variants and are pinned by closed
# forms instead.
# ---------------------------------------------------------------------------------------------------------
def _grads(seed, steps=5, shape=(6, 4)):
    g = hp.rng(seed)
    w0 = hp.normal(g, shape, np.float64)
    return w0, [hp.uniform(g, shape, 0.5, 2.0, np.float64) * np.where(g.random(shape) < 0.5, -1, 1) for _ in range(steps)]


def _run_oracle(rule, w0, grads, hyper, epoch=0):
    w, st = w0, [np.zeros_like(w0) for _ in range(3)]
    out = []
    for t, dw in enumerate(grads):
        w, st = oracle.optimizer_update(rule, w, dw, st, hyper, epoch=epoch, timestep=t)
        out.append(w)
    return out, st


def _run_torch(make_opt, w0, grads):
    pt = torch.tensor(w0.copy(), requires_grad=True)
    opt = make_opt([pt])
    out = []
    for dw in grads:
        pt.grad = torch.tensor(dw.copy())
        opt.step()
        out.append(pt.detach().numpy().copy())
    return out


@pytest.mark.parametrize("rule,hyper,make_opt", [
    ("vanilla_sgd", [0.05], lambda p: torch.optim.SGD(p, lr=0.05)),
    # s = momentum s + lr g, w -= s: torch's buffer times lr (annealing rate 0)
    ("momentum_sgd", [0.05, 0.0, 0.9], lambda p: torch.optim.SGD(p, lr=0.05, momentum=0.9)),
    # s = momentum s - lr g, w += -momentum s_old + (1 + momentum) s: torch's Nesterov step with s = -lr * buffer
    ("nesterov_momentum_sgd", [0.05, 0.0, 0.8], lambda p: torch.optim.SGD(p, lr=0.05, momentum=0.8, nesterov=True)),
    ("adagrad", [0.1, 1e-7], lambda p: torch.optim.Adagrad(p, lr=0.1, eps=1e-7)),
    ("rmsprop", [0.02, 0.1, 1e-7], lambda p: torch.optim.RMSprop(p, lr=0.02, alpha=0.9, eps=1e-7)),
    ("adadelta", [0.05, 1e-6], lambda p: torch.optim.Adadelta(p, lr=1.0, rho=0.95, eps=1e-6)),
])
def test_optimizers_that_coincide_with_torch(rule, hyper, make_opt):
    w0, grads = _grads(920)
    ours, _ = _run_oracle(rule, w0, grads, hyper)
    theirs = _run_torch(make_opt, w0, grads)
    for t, (a, b) in enumerate(zip(ours, theirs)):
        assert np.max(np.abs(a - b)) < 1e-12, (rule, t)


def test_adamax_matches_torch_in_the_small_epsilon_limit():
    """torch: u = max(beta2 u, |g| + eps), w -= lr / (1 - beta1^t) * m / u; the reference: u = max((1 - d2) u, |g|),
    w -= lr * m / (1 - (1 - d1)^t + eps) / (u + eps). Same recurrence for eps -> 0."""
    w0, grads = _grads(921)
    ours, _ = _run_oracle("adamax", w0, grads, [0.02, 0.1, 0.01, 1e-30])
    theirs = _run_torch(lambda p: torch.optim.Adamax(p, lr=0.02, betas=(0.9, 0.99), eps=1e-30), w0, grads)
    for a, b in zip(ours, theirs):
        assert np.max(np.abs(a - b)) < 1e-12


def test_annealed_learning_rate_of_the_momentum_optimizers():
    """calculate_learning_rate (MomentumSGDOptimizer.hpp:70-72): lr = init / (1 + annealing * epoch); at zero
    momentum-state the first step is w - lr g for both variants... Nesterov's is w - (1 + momentum) lr g."""
    w0, grads = _grads(922, steps=1)
    for epoch in (0, 3):
        lr = 0.1 / (1 + 0.5 * epoch)
        (w,), _ = _run_oracle("momentum_sgd", w0, grads, [0.1, 0.5, 0.9], epoch=epoch)
        assert np.max(np.abs(w - (w0 - lr * grads[0]))) < 1e-13
        (w,), _ = _run_oracle("nesterov_momentum_sgd", w0, grads, [0.1, 0.5, 0.9], epoch=epoch)
        assert np.max(np.abs(w - (w0 - 1.9 * lr * grads[0]))) < 1e-13


def test_nadam_first_step_closed_form_and_relation_to_adam():
    """From zero state at step 0 with eps -> 0: m = d1 g, v = d2 g^2, l1_corr = 1/d1, l1_next_corr = 1/(1-(1-d1)^2),
    l2_corr = 1/d2, so the step is lr sign(g) (1 + (1-d1)/(2-d1)). In general Nadam's numerator is
    d1 l1_corr g + (1-d1) l1_next_corr m where Adam's is l1_corr m, over the same denominator."""
    w0, grads = _grads(923, steps=3)
    d1, d2, lr = 0.2, 0.05, 0.01
    (w1, w2, w3), st = _run_oracle("nadam", w0, grads, [lr, d1, d2, 1e-30])
    assert np.max(np.abs(w1 - (w0 - lr * np.sign(grads[0]) * (1 + (1 - d1) / (2 - d1))))) < 1e-12
    # third step from the state after two steps, written out independently
    m = np.zeros_like(w0)
    v = np.zeros_like(w0)
    for dw in grads:
        m = (1 - d1) * m + d1 * dw
        v = (1 - d2) * v + d2 * dw * dw
    c1, c1n, c2 = 1 / (1 - (1 - d1) ** 3), 1 / (1 - (1 - d1) ** 4), 1 / (1 - (1 - d2) ** 3)
    assert np.max(np.abs(w3 - (w2 - lr * (d1 * c1 * grads[2] + (1 - d1) * c1n * m) / np.sqrt(c2 * v)))) < 1e-12
    assert hp.rel_err(st[0], m) < 1e-12 and hp.rel_err(st[1], v) < 1e-12


def test_amsgrad_keeps_the_running_maximum_and_has_no_bias_correction():
    """AMSGradOptimizer.hpp:48-66: w -= lr m / sqrt(max_t v_t + eps), m and v uncorrected. First step from zero
    state: lr d1 g / sqrt(d2 g^2 + eps); after a large gradient the denominator never shrinks."""
    shape = (5, 3)
    g = hp.rng(924)
    w0 = hp.normal(g, shape, np.float64)
    big = hp.uniform(g, shape, 5, 6, np.float64)
    small = [hp.uniform(g, shape, 0.1, 0.2, np.float64) for _ in range(4)]
    d1, d2, lr, eps = 0.1, 0.2, 0.01, 1e-8
    ws, st = _run_oracle("amsgrad", w0, [big] + small, [lr, d1, d2, eps])
    assert np.max(np.abs(ws[0] - (w0 - lr * d1 * big / np.sqrt(d2 * big * big + eps)))) < 1e-13
    vmax = d2 * big * big                      # v only decays from here on (small gradients): the maximum stays
    assert hp.rel_err(st[2], vmax) < 1e-13
    m = d1 * big
    w = ws[0]
    for t, dw in enumerate(small):
        m = (1 - d1) * m + d1 * dw
        w = w - lr * m / np.sqrt(vmax + eps)
        assert np.max(np.abs(ws[t + 1] - w)) < 1e-13


@pytest.mark.parametrize("rule,hyper", [("momentum_sgd", [1e-3, 1e-3, 0.9]), ("adagrad", [1e-2, 1e-5]), ("rmsprop", [1e-3, 1e-1, 1e-5]),
                                        ("adadelta", [5e-2, 1e-5]), ("adamax", [1e-3, 1e-1, 1e-3, 1e-5]),
                                        ("nadam", [1e-3, 1e-1, 1e-3, 1e-5]), ("amsgrad", [1e-3, 1e-1, 1e-3, 1e-5])])
def test_float32_optimizer_steps_track_float64(rule, hyper):
    """With the reference's default hyper-parameters, float32 steps stay within the float32 tolerance of float64 ones."""
    w0, grads = _grads(925, steps=3)
    w64, _ = _run_oracle(rule, w0, grads, hyper, epoch=2)
    w32, _ = _run_oracle(rule, w0.astype(np.float32), [dw.astype(np.float32) for dw in grads], hyper, epoch=2)
    assert hp.rel_err(w32[-1], w64[-1]) < 1e-4
