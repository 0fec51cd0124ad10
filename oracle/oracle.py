"""ctypes front-end of the CPU oracle (oracle/cattle_oracle.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py, always as the checker and never by the product path.

Tensors are numpy arrays of shape (N,H,W,C) in Fortran order, which is byte-for-byte the
reference's column-major Eigen layout (core/EigenProxy.hpp:43-64); matrices are Fortran-ordered
too. Every function returns new Fortran-ordered arrays.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcattle_oracle.so")

ACT_KINDS = {
    "identity": 0, "scaled": 1, "binary_step": 2, "sigmoid": 3, "tanh": 4, "softsign": 5,
    "softplus": 6, "relu": 7, "leaky_relu": 8, "elu": 9, "swish": 10,
}


def build(force=False):
    """Compile the oracle with its Makefile (g++)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError("oracle supports float32 and float64 only")


def _f(a, dtype):
    return np.asfortranarray(a, dtype=dtype)


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _ll(*v):
    return [ctypes.c_longlong(int(x)) for x in v]


def _call(name, dtype, *args):
    fn = getattr(lib(), "oracle_%s_%s" % (name, _sfx(dtype)))
    fn.restype = ctypes.c_int
    rc = fn(*args)
    if rc != 0:
        raise RuntimeError("oracle_%s failed with code %d" % (name, rc))


def num_threads():
    return int(lib().oracle_num_threads())


def set_num_threads(n):
    lib().oracle_set_num_threads(ctypes.c_int(int(n)))


def conv_out_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh):
    OH = (H - RH - (RH - 1) * dv + 2 * pv) // sv + 1
    OW = (W - RW - (RW - 1) * dh + 2 * ph) // sh + 1
    return OH, OW


def conv_forward(x, w, b, RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0, return_cache=False):
    dt = x.dtype
    x = _f(x, dt)
    N, H, W, C = x.shape
    K, F = w.shape
    assert K == RH * RW * C
    w = _f(w, dt)
    b = _f(np.reshape(b, (F,)), dt)
    OH, OW = conv_out_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    out = np.empty((N, OH, OW, F), dtype=dt, order="F")
    cache = np.empty((N * OH * OW, K), dtype=dt, order="F")
    _call("conv_forward", dt, *_ll(N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh),
          _p(x), _p(w), _p(b), _p(out), _p(cache))
    return (out, cache) if return_cache else out


def conv_backward(x_shape, cache, w, out_grad, RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0,
                  input_layer=False, wgrad=None, bgrad=None):
    """Returns (in_grad or None, wgrad, bgrad); wgrad/bgrad accumulate into the arrays passed in."""
    dt = out_grad.dtype
    N, H, W, C = x_shape
    K, F = w.shape
    w = _f(w, dt)
    out_grad = _f(out_grad, dt)
    cache = _f(cache, dt)
    wgrad = np.zeros((K, F), dtype=dt, order="F") if wgrad is None else wgrad
    bgrad = np.zeros((1, F), dtype=dt, order="F") if bgrad is None else bgrad
    in_grad = None if input_layer else np.empty((N, H, W, C), dtype=dt, order="F")
    _call("conv_backward", dt, *_ll(N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh),
          _p(cache), _p(w), _p(out_grad), _p(wgrad), _p(bgrad), _p(in_grad))
    return in_grad, wgrad, bgrad


def transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh):
    return ((IH - 1) * sv + RH + (RH - 1) * dv - 2 * pv, (IW - 1) * sh + RW + (RW - 1) * dh - 2 * ph)


def transconv_forward(x, w, b, F, RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0):
    """x (N,IH,IW,C); w [C x RH*RW*F]; b [1 x OH*OW*F]; returns (N,OH,OW,F)."""
    dt = x.dtype
    x = _f(x, dt)
    N, IH, IW, C = x.shape
    assert w.shape == (C, RH * RW * F)
    OH, OW = transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh)
    w = _f(w, dt)
    b = _f(np.reshape(b, (OH * OW * F,)), dt)
    out = np.empty((N, OH, OW, F), dtype=dt, order="F")
    _call("transconv_forward", dt, *_ll(N, IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh), _p(x), _p(w), _p(b), _p(out))
    return out


def transconv_backward(x, w, out_grad, RH=3, RW=3, pv=1, ph=1, sv=1, sh=1, dv=0, dh=0, input_layer=False, wgrad=None,
                       bgrad=None):
    """Returns (in_grad or None, wgrad, bgrad); wgrad/bgrad accumulate into the arrays passed in."""
    dt = x.dtype
    x, w, out_grad = _f(x, dt), _f(w, dt), _f(out_grad, dt)
    N, IH, IW, C = x.shape
    F = out_grad.shape[3]
    wgrad = np.zeros(w.shape, dtype=dt, order="F") if wgrad is None else wgrad
    bgrad = np.zeros((1, out_grad.size // N), dtype=dt, order="F") if bgrad is None else bgrad
    in_grad = None if input_layer else np.empty(x.shape, dtype=dt, order="F")
    _call("transconv_backward", dt, *_ll(N, IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh), _p(x), _p(w), _p(out_grad),
          _p(wgrad), _p(bgrad), _p(in_grad))
    return in_grad, wgrad, bgrad


def dense_forward(x, w, b):
    dt = x.dtype
    N = x.shape[0]
    V, O = w.shape
    x = _f(x, dt)
    assert x.size == N * V
    out = np.empty((N, O), dtype=dt, order="F")
    w = _f(w, dt)
    b = _f(np.reshape(b, (O,)), dt)
    _call("dense_forward", dt, *_ll(N, V, O), _p(x), _p(w), _p(b), _p(out))
    return out


def dense_backward(x, w, out_grad, input_layer=False, wgrad=None, bgrad=None):
    dt = x.dtype
    N = x.shape[0]
    V, O = w.shape
    x = _f(x, dt)
    out_grad = _f(out_grad, dt)
    wgrad = np.zeros((V, O), dtype=dt, order="F") if wgrad is None else wgrad
    bgrad = np.zeros((1, O), dtype=dt, order="F") if bgrad is None else bgrad
    in_grad = None if input_layer else np.empty(x.shape, dtype=dt, order="F")
    w = _f(w, dt)
    _call("dense_backward", dt, *_ll(N, V, O), _p(x), _p(w), _p(out_grad), _p(wgrad), _p(bgrad), _p(in_grad))
    return in_grad, wgrad, bgrad


def bn_forward(x, gamma, beta, avg_mean, avg_inv_sd, stats_init, training, per_channel=True, decay=0.1,
               eps=1e-5):
    """gamma/beta/avg_* are 1-D arrays over the statistics groups; avg_* are updated in place.
    Returns (out, std_cache, inv_sd_cache)."""
    dt = x.dtype
    x = _f(x, dt)
    N = x.shape[0]
    groups = x.shape[-1] if per_channel else x.size // N
    L = x.size // groups
    out = np.empty(x.shape, dtype=dt, order="F")
    std_cache = np.empty(x.shape, dtype=dt, order="F")
    inv_sd = np.zeros((groups,), dtype=dt)
    assert avg_mean.dtype == dt and avg_inv_sd.dtype == dt and avg_mean.flags.c_contiguous
    gamma, beta = _f(gamma, dt), _f(beta, dt)
    _call("bn_forward", dt, *_ll(groups, L), _p(x), _p(gamma), _p(beta), _p(avg_mean),
          _p(avg_inv_sd), ctypes.c_int(int(stats_init)), ctypes.c_int(int(training)), ctypes.c_double(decay),
          ctypes.c_double(eps), _p(out), _p(std_cache), _p(inv_sd))
    return out, std_cache, inv_sd


def bn_backward(out_grad, gamma, std_cache, inv_sd, per_channel=True, input_layer=False, gamma_grad=None,
                beta_grad=None):
    dt = out_grad.dtype
    g = _f(out_grad, dt)
    N = g.shape[0]
    groups = g.shape[-1] if per_channel else g.size // N
    L = g.size // groups
    gamma_grad = np.zeros((groups,), dtype=dt) if gamma_grad is None else gamma_grad
    beta_grad = np.zeros((groups,), dtype=dt) if beta_grad is None else beta_grad
    dx = None if input_layer else np.empty(g.shape, dtype=dt, order="F")
    gamma, std_cache, inv_sd = _f(gamma, dt), _f(std_cache, dt), _f(inv_sd, dt)
    _call("bn_backward", dt, *_ll(groups, L), _p(g), _p(gamma), _p(std_cache), _p(inv_sd), _p(gamma_grad),
          _p(beta_grad), _p(dx))
    return dx, gamma_grad, beta_grad


def act_forward(kind, x, p=0.0):
    dt = x.dtype
    x = _f(x, dt)
    y = np.empty(x.shape, dtype=dt, order="F")
    _call("act_forward", dt, ctypes.c_int(ACT_KINDS[kind]), *_ll(x.size), ctypes.c_double(p), _p(x), _p(y))
    return y


def act_backward(kind, x, y, g, p=0.0):
    dt = x.dtype
    x, y, g = _f(x, dt), _f(y, dt), _f(g, dt)
    dx = np.empty(x.shape, dtype=dt, order="F")
    _call("act_backward", dt, ctypes.c_int(ACT_KINDS[kind]), *_ll(x.size), ctypes.c_double(p), _p(x), _p(y),
          _p(g), _p(dx))
    return dx


def softmax_forward(x, eps=1e-5):
    dt = x.dtype
    x = _f(x, dt)
    N = x.shape[0]
    y = np.empty(x.shape, dtype=dt, order="F")
    _call("softmax_forward", dt, *_ll(N, x.size // N), ctypes.c_double(eps), _p(x), _p(y))
    return y


def softmax_backward(y, g):
    dt = y.dtype
    y, g = _f(y, dt), _f(g, dt)
    N = y.shape[0]
    dx = np.empty(y.shape, dtype=dt, order="F")
    _call("softmax_backward", dt, *_ll(N, y.size // N), _p(y), _p(g), _p(dx))
    return dx


def _param_act(name, x, param, g=None, input_layer=False, param_grad=None):
    dt = x.dtype
    x = _f(x, dt)
    N = x.shape[0]
    V = x.size // N
    param = _f(np.reshape(param, (V,)), dt)
    if g is None:
        y = np.empty(x.shape, dtype=dt, order="F")
        _call(name + "_forward", dt, *_ll(N, V), _p(param), _p(x), _p(y))
        return y
    g = _f(g, dt)
    param_grad = np.zeros((V,), dtype=dt) if param_grad is None else param_grad
    dx = None if input_layer else np.empty(x.shape, dtype=dt, order="F")
    _call(name + "_backward", dt, *_ll(N, V), _p(param), _p(x), _p(g), _p(param_grad), _p(dx))
    return dx, param_grad


def prelu_forward(x, alpha):
    return _param_act("prelu", x, alpha)


def prelu_backward(x, alpha, g, param_grad=None):
    return _param_act("prelu", x, alpha, g, False, param_grad)


def pswish_forward(x, beta):
    return _param_act("pswish", x, beta)


def pswish_backward(x, beta, g, input_layer=False, param_grad=None):
    return _param_act("pswish", x, beta, g, input_layer, param_grad)


def pool_out_dims(H, W, RH, RW, sv, sh):
    return (H - RH) // sv + 1, (W - RW) // sh + 1


def maxpool_forward(x, RH=2, RW=2, sv=2, sh=2):
    """Returns (out, inds) with inds of shape (OH*OW, C*N), uint32, as the reference caches them."""
    dt = x.dtype
    x = _f(x, dt)
    N, H, W, C = x.shape
    OH, OW = pool_out_dims(H, W, RH, RW, sv, sh)
    out = np.empty((N, OH, OW, C), dtype=dt, order="F")
    inds = np.empty((OH * OW, C * N), dtype=np.uint32)
    _call("maxpool_forward", dt, *_ll(N, H, W, C, RH, RW, sv, sh), _p(x), _p(out), _p(inds))
    return out, inds


def maxpool_backward(x_shape, out_grad, inds, RH=2, RW=2, sv=2, sh=2):
    dt = out_grad.dtype
    N, H, W, C = x_shape
    g = _f(out_grad, dt)
    inds = np.ascontiguousarray(inds, dtype=np.uint32)
    dx = np.empty((N, H, W, C), dtype=dt, order="F")
    _call("maxpool_backward", dt, *_ll(N, H, W, C, RH, RW, sv, sh), _p(g), _p(inds), _p(dx))
    return dx


def meanpool_forward(x, RH=2, RW=2, sv=2, sh=2):
    dt = x.dtype
    x = _f(x, dt)
    N, H, W, C = x.shape
    OH, OW = pool_out_dims(H, W, RH, RW, sv, sh)
    out = np.empty((N, OH, OW, C), dtype=dt, order="F")
    _call("meanpool_forward", dt, *_ll(N, H, W, C, RH, RW, sv, sh), _p(x), _p(out))
    return out


def meanpool_backward(x_shape, out_grad, RH=2, RW=2, sv=2, sh=2):
    dt = out_grad.dtype
    N, H, W, C = x_shape
    g = _f(out_grad, dt)
    dx = np.empty((N, H, W, C), dtype=dt, order="F")
    _call("meanpool_backward", dt, *_ll(N, H, W, C, RH, RW, sv, sh), _p(g), _p(dx))
    return dx


def splitmix64_output(seed, index):
    fn = lib().oracle_splitmix64_output
    fn.restype = ctypes.c_ulonglong
    return int(fn(ctypes.c_ulonglong(seed), ctypes.c_ulonglong(index)))


def dropout_uniforms(seed, pass_index, shape, dtype):
    """The uniform numbers of training pass `pass_index` of a dropout layer seeded with `seed`, in the shape of the batch."""
    u = np.empty(shape, dtype=dtype, order="F")
    _call("dropout_uniforms", np.dtype(dtype), ctypes.c_ulonglong(seed), ctypes.c_ulonglong(pass_index), *_ll(u.size), _p(u))
    return u


def dropout_apply(x, u, prob, eps=1e-5):
    """x times the dropout mask of the uniforms u (layer/DropoutLayer.hpp:78-82, :95)."""
    dt = x.dtype
    x, u = _f(x, dt), _f(u, dt)
    y = np.empty(x.shape, dtype=dt, order="F")
    _call("dropout_apply", dt, *_ll(x.size), ctypes.c_double(prob), ctypes.c_double(eps), _p(u), _p(x), _p(y))
    return y


def broadcast_forward(x, bh, bw, bc):
    dt = x.dtype
    x = _f(x, dt)
    N, H, W, C = x.shape
    out = np.empty((N, H * bh, W * bw, C * bc), dtype=dt, order="F")
    _call("broadcast_forward", dt, *_ll(N, H, W, C, bh, bw, bc), _p(x), _p(out))
    return out


def broadcast_backward(x_shape, out_grad, bh, bw, bc):
    dt = out_grad.dtype
    N, H, W, C = x_shape
    g = _f(out_grad, dt)
    dx = np.empty((N, H, W, C), dtype=dt, order="F")
    _call("broadcast_backward", dt, *_ll(N, H, W, C, bh, bw, bc), _p(g), _p(dx))
    return dx


LOSS_KINDS = {"squared": 0, "softmax_cross_entropy": 1, "absolute": 2, "binary_cross_entropy": 3, "cross_entropy": 4,
              "kullback_leibler": 5, "hinge": 6, "squared_hinge": 7, "multi_label_hinge": 8,
              "squared_multi_label_hinge": 9, "multi_label_log": 10}
LOSS_NEGATED = 0x100        # the loss wrapped in NegatedLoss (loss/NegatedLoss.hpp:41-46)


def _loss_kind(kind, negated):
    return ctypes.c_int(LOSS_KINDS[kind] | (LOSS_NEGATED if negated else 0))


def _loss_dims(out, sequential):
    N = out.shape[0]
    Ts = out.shape[1] if sequential else 1
    return N, Ts, out.size // (N * Ts)


def loss_function(kind, out, obj, eps=1e-5, sequential=False, negated=False):
    """Per-sample losses (summed over time steps when sequential: out is then (N, T, ...))."""
    dt = out.dtype
    out, obj = _f(out, dt), _f(obj, dt)
    N, Ts, V = _loss_dims(out, sequential)
    losses = np.empty((N,), dtype=dt)
    _call("loss_function", dt, _loss_kind(kind, negated), *_ll(N, Ts, V), ctypes.c_double(eps), _p(out), _p(obj),
          _p(losses))
    return losses


def loss_d_function(kind, out, obj, eps=1e-5, scale=1.0, sequential=False, negated=False):
    dt = out.dtype
    out, obj = _f(out, dt), _f(obj, dt)
    N, Ts, V = _loss_dims(out, sequential)
    grad = np.empty(out.shape, dtype=dt, order="F")
    _call("loss_d_function", dt, _loss_kind(kind, negated), *_ll(N, Ts, V), ctypes.c_double(eps),
          ctypes.c_double(scale), _p(out), _p(obj), _p(grad))
    return grad


def regularization(values, l1=0.0, l2=0.0):
    """(penalty, gradient) of a parameter's regularization at `values`: L1 (l1, 0), L2 (0, l2) or elastic net."""
    dt = values.dtype
    v = _f(values, dt)
    grad = np.empty(v.shape, dtype=dt, order="F")
    penalty = np.zeros((1,), dtype=dt)
    _call("regularization", dt, *_ll(v.size), ctypes.c_double(l1), ctypes.c_double(l2), _p(v), _p(penalty), _p(grad))
    return float(penalty[0]), grad


def constrain(matrix, clip=0.0, max_l1_norm=0.0, max_l2_norm=0.0):
    """The constraints StandardParameters enforces on its values in set_values and on its gradient in accumulate_grad
    (parameters/StandardParameters.hpp:105-123), in the arithmetic of the matrix's type and in the reference's order:
    enforce_clip_constraint (:150-156) clips to [-clip, clip]; enforce_l1_norm_constraint (:163-169) scales by
    max_l1_norm / matrix.norm() - Eigen's norm() is the Euclidean one - if that norm exceeds the limit;
    enforce_l2_norm_constraint (:176-182) scales by max_l2_norm / matrix.squaredNorm() if the squared norm exceeds the
    limit. A limit takes effect if NumericUtils::decidedly_greater(limit, 0) (core/NumericUtils.hpp:42-65: greater than
    zero and not within the type's epsilon of it). Returns a new matrix."""
    dt = matrix.dtype
    m = np.array(matrix, dtype=dt, order="F", copy=True)
    eps = np.finfo(dt).eps

    def on(limit):
        return dt.type(limit) > eps

    if on(clip):
        c = dt.type(clip)
        m = np.where(m > c, c, np.where(m < -c, -c, m)).astype(dt)
    if on(max_l1_norm):
        norm = np.sqrt(np.sum(m * m, dtype=dt), dtype=dt)
        if norm > dt.type(max_l1_norm):
            m = (m * (dt.type(max_l1_norm) / norm)).astype(dt)
    if on(max_l2_norm):
        sq = np.sum(m * m, dtype=dt)
        if sq > dt.type(max_l2_norm):
            m = (m * (dt.type(max_l2_norm) / sq)).astype(dt)
    return np.asfortranarray(m)


def sgd_update(values, grad, lr=1e-3):
    """Returns the updated values (the inputs are left alone)."""
    dt = values.dtype
    new = np.array(values, dtype=dt, order="F", copy=True)
    grad = _f(grad, dt)
    _call("sgd_update", dt, *_ll(new.size), ctypes.c_double(lr), _p(grad), _p(new))
    return new


def adam_update(values, grad, m, v, timestep, lr=1e-3, l1_decay=1e-1, l2_decay=1e-3, eps=1e-5):
    """Returns (values, m, v) after one step; m and v are the moving averages before it."""
    dt = values.dtype
    new, m, v = (np.array(a, dtype=dt, order="F", copy=True) for a in (values, m, v))
    grad = _f(grad, dt)
    _call("adam_update", dt, *_ll(new.size), ctypes.c_double(lr), ctypes.c_double(l1_decay), ctypes.c_double(l2_decay),
          ctypes.c_double(eps), *_ll(timestep), _p(grad), _p(m), _p(v), _p(new))
    return new, m, v


OPTIMIZERS = {"vanilla_sgd": 0, "momentum_sgd": 1, "nesterov_momentum_sgd": 2, "adagrad": 3, "rmsprop": 4, "adadelta": 5,
              "adam": 6, "adamax": 7, "nadam": 8, "amsgrad": 9}


def optimizer_update(rule, values, grad, states, hyper, epoch=0, timestep=0):
    """One _update_params of optimizer `rule` on one parameter matrix. states: three matrices (unused ones are
    ignored); hyper: the optimizer's constructor arguments in their order. Returns (values, [s0, s1, s2])."""
    dt = values.dtype
    new = np.array(values, dtype=dt, order="F", copy=True)
    st = [np.array(s, dtype=dt, order="F", copy=True) for s in states]
    grad = _f(grad, dt)
    h = (ctypes.c_double * 4)(*(list(hyper) + [0.0] * (4 - len(hyper))))
    _call("optimizer_update", dt, ctypes.c_int(OPTIMIZERS[rule]), h, *_ll(epoch, timestep, new.size), _p(grad), _p(st[0]),
          _p(st[1]), _p(st[2]), _p(new))
    return new, st
