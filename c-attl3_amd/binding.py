"""ctypes binding of libcattle_hip.so plus thin layer classes that mirror cattle::Layer.

The classes carry the reference's names and method names (pass_forward, pass_back, get_params,
set_input_layer, empty_cache, clone, clone_with_shared_params: core/Layer.hpp:47-137) so that tests
read like the reference's. Host tensors are numpy arrays of shape (N,H,W,C) in Fortran order, i.e.
the reference's column-major Eigen buffers; DeviceTensor keeps a tensor resident in HBM between
layers. There is no host fallback: without the built library or without an MI355X every call raises.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# CATTLE_HIP_LIBRARY overrides the location of the built library (e.g. an experimental build)
LIB_PATH = os.environ.get("CATTLE_HIP_LIBRARY") or os.path.join(_HERE, "libcattle_hip.so")

F32, F64 = 0, 1
HOST, DEVICE = 0, 1
POOL_MAX, POOL_MEAN = 0, 1
ACT = {
    "identity": 0, "scaled": 1, "binary_step": 2, "sigmoid": 3, "tanh": 4, "softsign": 5, "softplus": 6,
    "relu": 7, "leaky_relu": 8, "elu": 9, "swish": 10, "softmax": 11, "prelu": 12, "pswish": 13,
}

# every symbol include/cattle_hip.h declares
EXPORTS = [
    "cattle_hip_init", "cattle_hip_last_error", "cattle_hip_synchronize", "cattle_hip_alloc", "cattle_hip_free", "cattle_hip_trim", "cattle_hip_memory_info",
    "cattle_hip_upload", "cattle_hip_download", "cattle_hip_fill_zero", "cattle_hip_timer_create",
    "cattle_hip_timer_destroy", "cattle_hip_timer_start", "cattle_hip_timer_stop", "cattle_hip_conv_create",
    "cattle_hip_transconv_create", "cattle_hip_dense_create", "cattle_hip_batchnorm_create", "cattle_hip_batchnorm_get_stats_initialized",
    "cattle_hip_batchnorm_set_stats_initialized", "cattle_hip_activation_create", "cattle_hip_pool_create",
    "cattle_hip_convlstm_set_multiplicative_integration", "cattle_hip_convlstm_fused_steps", "cattle_hip_layer_param_set_regularization",
    "cattle_hip_layer_param_regularization_penalty", "cattle_hip_dropout_create", "cattle_hip_reshape_create", "cattle_hip_broadcast_create",
    "cattle_hip_layer_clone", "cattle_hip_layer_destroy", "cattle_hip_layer_input_dims",
    "cattle_hip_layer_output_dims", "cattle_hip_layer_is_input_layer", "cattle_hip_layer_set_input_layer",
    "cattle_hip_layer_empty_cache", "cattle_hip_layer_forward", "cattle_hip_layer_backward",
    "cattle_hip_layer_num_params", "cattle_hip_layer_param_shape", "cattle_hip_layer_set_param_values",
    "cattle_hip_layer_get_param_values", "cattle_hip_layer_get_param_grad", "cattle_hip_layer_reset_param_grad",
    "cattle_hip_maxpool_indices", "cattle_hip_loss_function", "cattle_hip_loss_d_function",
    "cattle_hip_layer_param_optimizer_update", "cattle_hip_layer_param_optimizer_step", "cattle_hip_optimizer_step_many", "cattle_hip_layer_param_sgd_update", "cattle_hip_layer_param_adam_update",
    "cattle_hip_layer_param_reset_optimizer_state", "cattle_hip_convlstm_create", "cattle_hip_convlstm_propagate",
    "cattle_hip_convlstm_backpropagate", "cattle_hip_convlstm_set_kernel_values", "cattle_hip_convlstm_get_kernel_values",
    "cattle_hip_convlstm_get_kernel_grad", "cattle_hip_conv_forward_noalloc", "cattle_hip_static_scratch_bytes",
    "cattle_hip_fused_create", "cattle_hip_fused_last_mode", "cattle_hip_graph_begin_capture", "cattle_hip_graph_end_capture",
    "cattle_hip_graph_launch", "cattle_hip_graph_destroy", "cattle_hip_layer_param_set_constraints",
]


class CattleHipError(RuntimeError):
    def __init__(self, code, message):
        RuntimeError.__init__(self, "cattle_hip error %d: %s" % (code, message))
        self.code = code


def build():
    """Compile libcattle_hip.so for gfx950 with the package Makefile (hipcc cross-compiles)."""
    subprocess.check_call(["make", "-s", "-j4", "-C", _HERE])


_lib = None


def lib():
    """Loads the built library; raises if it has not been built (there is no other code path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CattleHipError(-1, "libcattle_hip.so is not built: run __graft_entry__.build() or make -C c-attl3_amd")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.cattle_hip_last_error.restype = ctypes.c_char_p
        for name in EXPORTS:
            if name != "cattle_hip_last_error":
                getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _check(rc):
    if rc != 0:
        raise CattleHipError(rc, lib().cattle_hip_last_error().decode("utf-8", "replace"))


def init(device=0):
    _check(lib().cattle_hip_init(ctypes.c_int(device)))


def memory_info():
    """(free, total) device memory in bytes; buffers idling in the library's pool count as used."""
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    _check(lib().cattle_hip_memory_info(ctypes.byref(free), ctypes.byref(total)))
    return int(free.value), int(total.value)


def trim():
    """Returns the device memory that released DeviceTensors left idle in the library's pool to the driver."""
    _check(lib().cattle_hip_trim())


def synchronize():
    _check(lib().cattle_hip_synchronize())


def _dtype_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return F32
    if dtype == np.float64:
        return F64
    raise TypeError("Scalar must be float32 or float64")


def _sz(v):
    return ctypes.c_size_t(int(v))


class DeviceTensor(object):
    """A tensor resident in device memory, in the reference's column-major layout."""

    def __init__(self, shape, dtype):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        _check(lib().cattle_hip_alloc(ctypes.byref(p), _sz(self.nbytes)))
        self.ptr = p

    @staticmethod
    def from_host(a):
        a = np.asfortranarray(a)
        t = DeviceTensor(a.shape, a.dtype)
        _check(lib().cattle_hip_upload(t.ptr, ctypes.c_void_p(a.ctypes.data), _sz(t.nbytes)))
        return t

    def to_host(self):
        a = np.empty(self.shape, dtype=self.dtype, order="F")
        _check(lib().cattle_hip_download(ctypes.c_void_p(a.ctypes.data), self.ptr, _sz(self.nbytes)))
        return a

    def free(self):
        if self.ptr is not None and self.ptr.value:
            _check(lib().cattle_hip_free(self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def static_scratch_bytes():
    """Size of the fixed device array that conv_forward_noalloc takes its scratch memory from."""
    v = ctypes.c_size_t()
    _check(lib().cattle_hip_static_scratch_bytes(ctypes.byref(v)))
    return int(v.value)


def conv_forward_noalloc(x, weights, bias, out, receptor_height=3, receptor_width=3, vertical_padding=1, horizontal_padding=1,
                         vertical_stride=1, horizontal_stride=1, vertical_dilation=0, horizontal_dilation=0):
    """ConvKernelLayer::pass_forward on DeviceTensors the caller owns, through the entry point that allocates nothing:
    x (N, H, W, C), weights (RH*RW*C, F), bias (1, F) or None, out (N, OH, OW, F)."""
    if len(x.shape) != 4 or len(weights.shape) != 2 or len(out.shape) != 4:
        raise ValueError("x and out must be (N, H, W, C) tensors, weights a matrix")
    N, H, W, C = x.shape
    F = weights.shape[1]
    # the entry point takes raw addresses and cannot know the buffers' sizes: every extent is checked here
    drh = receptor_height + (receptor_height - 1) * vertical_dilation
    drw = receptor_width + (receptor_width - 1) * horizontal_dilation
    if min(receptor_height, receptor_width, vertical_stride, horizontal_stride) < 1 or min(
            vertical_padding, horizontal_padding, vertical_dilation, horizontal_dilation) < 0:
        raise ValueError("receptor and strides must be positive, paddings and dilations non-negative")
    if H + 2 * vertical_padding < drh or W + 2 * horizontal_padding < drw:
        raise ValueError("dilated receptor larger than the padded input")
    OH = (H + 2 * vertical_padding - drh) // vertical_stride + 1          # ConvKernelLayer.hpp:194-197
    OW = (W + 2 * horizontal_padding - drw) // horizontal_stride + 1
    if weights.shape[0] != receptor_height * receptor_width * C:
        raise ValueError("weights must have receptor_height * receptor_width * channels = %d rows, not %d"
                         % (receptor_height * receptor_width * C, weights.shape[0]))
    if bias is not None and tuple(bias.shape) != (1, F):
        raise ValueError("bias must be a (1, %d) matrix, not %s" % (F, tuple(bias.shape)))
    if tuple(out.shape) != (N, OH, OW, F):
        raise ValueError("out must be %s, not %s" % ((N, OH, OW, F), tuple(out.shape)))
    for name, t in (("weights", weights), ("bias", bias), ("out", out)):
        if t is not None and np.dtype(t.dtype) != np.dtype(x.dtype):
            raise ValueError("%s is %s, x is %s" % (name, np.dtype(t.dtype), np.dtype(x.dtype)))
    _check(lib().cattle_hip_conv_forward_noalloc(
        _dtype_code(x.dtype), _sz(N), _sz(H), _sz(W), _sz(C), _sz(F), _sz(receptor_height), _sz(receptor_width),
        _sz(vertical_padding), _sz(horizontal_padding), _sz(vertical_stride), _sz(horizontal_stride), _sz(vertical_dilation),
        _sz(horizontal_dilation), x.ptr, weights.ptr, None if bias is None else bias.ptr, out.ptr))


class Timer(object):
    def __init__(self):
        self.h = ctypes.c_void_p()
        _check(lib().cattle_hip_timer_create(ctypes.byref(self.h)))

    def start(self):
        _check(lib().cattle_hip_timer_start(self.h))

    def stop(self):
        ms = ctypes.c_float()
        _check(lib().cattle_hip_timer_stop(self.h, ctypes.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            lib().cattle_hip_timer_destroy(self.h)
        except Exception:
            pass


class Parameters(object):
    """View of one parameter matrix of a layer (core/Parameters.hpp:15-95)."""

    def __init__(self, layer, index):
        self._layer, self._index = layer, index
        r, c, o = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_int()
        _check(lib().cattle_hip_layer_param_shape(layer._h, _sz(index), ctypes.byref(r), ctypes.byref(c), ctypes.byref(o)))
        self._rows, self._cols, self._opt = int(r.value), int(c.value), bool(o.value)

    def get_rows(self):
        return self._rows

    def get_cols(self):
        return self._cols

    def are_optimizable(self):
        return self._opt

    def get_values(self):
        a = np.empty((self._rows, self._cols), dtype=self._layer.dtype, order="F")
        _check(lib().cattle_hip_layer_get_param_values(self._layer._h, _sz(self._index), ctypes.c_void_p(a.ctypes.data), HOST))
        return a

    def set_values(self, values):
        a = np.asfortranarray(values, dtype=self._layer.dtype)
        if a.shape != (self._rows, self._cols):
            raise ValueError("expected a %dx%d matrix" % (self._rows, self._cols))
        _check(lib().cattle_hip_layer_set_param_values(self._layer._h, _sz(self._index), ctypes.c_void_p(a.ctypes.data), HOST))

    def get_grad(self):
        a = np.empty((self._rows, self._cols), dtype=self._layer.dtype, order="F")
        _check(lib().cattle_hip_layer_get_param_grad(self._layer._h, _sz(self._index), ctypes.c_void_p(a.ctypes.data), HOST))
        return a

    def reset_grad(self):
        _check(lib().cattle_hip_layer_reset_param_grad(self._layer._h, _sz(self._index)))

    def optimizer_update(self, optimizer, hyper, epoch=0, timestep=0):
        """<Name>Optimizer::_update_params on the device; optimizer is a key of OPTIMIZERS, hyper the reference
        optimizer's constructor arguments in their order (see include/cattle_hip.h)."""
        h = _hyper_array(tuple(hyper))
        _check(lib().cattle_hip_layer_param_optimizer_update(self._layer._h, _sz(self._index), ctypes.c_int(OPTIMIZERS[optimizer]),
                                                             h, _sz(epoch), _sz(timestep)))

    def optimizer_step(self, optimizer, hyper, epoch=0, timestep=0):
        """optimizer_update followed by reset_grad (optimizer/SGDOptimizer.hpp:64, :68-70) as one kernel."""
        h = _hyper_array(tuple(hyper))
        _check(lib().cattle_hip_layer_param_optimizer_step(self._layer._h, _sz(self._index), ctypes.c_int(OPTIMIZERS[optimizer]),
                                                           h, _sz(epoch), _sz(timestep)))

    def set_regularization(self, l1_lambda=0.0, l2_lambda=0.0):
        """The parameter's ParameterRegularization: L1 (l1, 0), L2 (0, l2), elastic net (l1, l2), none (0, 0)
        (parameter_regularization/*.hpp); optimizer_step then regularizes before it updates."""
        _check(lib().cattle_hip_layer_param_set_regularization(self._layer._h, _sz(self._index), ctypes.c_double(l1_lambda),
                                                               ctypes.c_double(l2_lambda)))

    def set_constraints(self, value_clip=0.0, value_max_l1_norm=0.0, value_max_l2_norm=0.0, grad_clip=0.0, grad_max_l1_norm=0.0,
                        grad_max_l2_norm=0.0):
        """The constraints of parameters/StandardParameters.hpp:61-76 on device-resident parameters; 0 = off."""
        _check(lib().cattle_hip_layer_param_set_constraints(self._layer._h, _sz(self._index), *[ctypes.c_double(v) for v in (
            value_clip, value_max_l1_norm, value_max_l2_norm, grad_clip, grad_max_l1_norm, grad_max_l2_norm)]))

    def get_regularization_penalty(self):
        """Parameters::get_regularization_penalty (parameters/StandardParameters.hpp:128-132)."""
        v = ctypes.c_double()
        _check(lib().cattle_hip_layer_param_regularization_penalty(self._layer._h, _sz(self._index), ctypes.byref(v)))
        return float(v.value)

    def sgd_update(self, learning_rate=1e-3):
        """VanillaSGDOptimizer::_update_params on the device (optimizer/VanillaSGDOptimizer.hpp:38-43)."""
        _check(lib().cattle_hip_layer_param_sgd_update(self._layer._h, _sz(self._index), ctypes.c_double(learning_rate)))

    def adam_update(self, timestep, learning_rate=1e-3, l1_decay=1e-1, l2_decay=1e-3, epsilon=1e-5):
        """AdamOptimizer::_update_params on the device; defaults of optimizer/AdamOptimizer.hpp:40-42."""
        _check(lib().cattle_hip_layer_param_adam_update(self._layer._h, _sz(self._index), ctypes.c_double(learning_rate),
                                                        ctypes.c_double(l1_decay), ctypes.c_double(l2_decay),
                                                        ctypes.c_double(epsilon), _sz(timestep)))

    def reset_optimizer_state(self):
        """AdamOptimizer::_fit: zero the moving averages."""
        _check(lib().cattle_hip_layer_param_reset_optimizer_state(self._layer._h, _sz(self._index)))


LOSS = {"squared": 0, "softmax_cross_entropy": 1, "absolute": 2, "binary_cross_entropy": 3, "cross_entropy": 4,
        "kullback_leibler": 5, "hinge": 6, "squared_hinge": 7, "multi_label_hinge": 8, "squared_multi_label_hinge": 9,
        "multi_label_log": 10}
LOSS_NEGATED = 0x100        # OR-ed into a kind: the loss wrapped in NegatedLoss (loss/NegatedLoss.hpp:41-46)
_HYPER_ARRAYS = {}


class ParameterList(object):
    """The optimizable parameters of a network, updated and reset together (optimizer_step of each, one launch per
    sixteen): SGDOptimizer::_train's loops over get_all_unique_params (optimizer/SGDOptimizer.hpp:58-70)."""

    def __init__(self, params):
        self._params = [p for p in params if p.are_optimizable()]
        n = len(self._params)
        self._layers = (ctypes.c_void_p * n)(*[p._layer._h for p in self._params])
        self._indices = (ctypes.c_size_t * n)(*[p._index for p in self._params])

    def __len__(self):
        return len(self._params)

    def optimizer_step(self, optimizer, hyper, epoch=0, timestep=0):
        _check(lib().cattle_hip_optimizer_step_many(self._layers, self._indices, _sz(len(self._params)),
                                                    ctypes.c_int(OPTIMIZERS[optimizer]), _hyper_array(tuple(hyper)),
                                                    _sz(epoch), _sz(timestep)))


def _hyper_array(hyper):
    """The four-entry hyper-parameter array of an optimizer call (read-only on the C side, so one per value set)."""
    h = _HYPER_ARRAYS.get(hyper)
    if h is None:
        h = _HYPER_ARRAYS[hyper] = (ctypes.c_double * 4)(*(list(hyper) + [0.0] * (4 - len(hyper))))
    return h
OPTIMIZERS = {"vanilla_sgd": 0, "momentum_sgd": 1, "nesterov_momentum_sgd": 2, "adagrad": 3, "rmsprop": 4, "adadelta": 5,
              "adam": 6, "adamax": 7, "nadam": 8, "amsgrad": 9}


def _loss_args(out, obj, sequential):
    if isinstance(out, DeviceTensor) != isinstance(obj, DeviceTensor):
        raise TypeError("out and obj must both be numpy arrays or both DeviceTensors")
    if not isinstance(out, DeviceTensor):
        out = np.asfortranarray(out)
        obj = np.asfortranarray(obj, dtype=out.dtype)
    if tuple(out.shape) != tuple(obj.shape):
        raise ValueError("out and obj dimensions differ")          # assert(out.dimensions() == obj.dimensions())
    batch = out.shape[0]
    steps = out.shape[1] if sequential else 1
    size = int(np.prod(out.shape[1:])) // steps
    dev = isinstance(out, DeviceTensor)
    ptr = (lambda t: t.ptr) if dev else (lambda a: ctypes.c_void_p(a.ctypes.data))
    return out, obj, batch, steps, size, (DEVICE if dev else HOST), ptr


def _loss_kind(kind, negated):
    return ctypes.c_int(LOSS[kind] | (LOSS_NEGATED if negated else 0))


def loss_function(kind, out, obj, epsilon=1e-5, sequential=False, negated=False):
    """Loss::function: the per-sample losses of a batch as a numpy vector (loss/UniversalLoss.hpp:37-41, :99-110).
    out/obj are numpy arrays or DeviceTensors of shape (N, ...) or, if sequential, (N, T, ...); `negated` is the
    loss wrapped in NegatedLoss."""
    out, obj, batch, steps, size, space, ptr = _loss_args(out, obj, sequential)
    losses = np.empty((batch,), dtype=out.dtype)
    _check(lib().cattle_hip_loss_function(_dtype_code(out.dtype), _loss_kind(kind, negated), ptr(out), space, ptr(obj), space,
                                          _sz(batch), _sz(steps), _sz(size), ctypes.c_double(epsilon),
                                          ctypes.c_void_p(losses.ctypes.data), HOST))
    return losses


def loss_d_function(kind, out, obj, epsilon=1e-5, scale=1.0, sequential=False, negated=False):
    """Loss::d_function times scale (loss/UniversalLoss.hpp:42-46, :111-125); returns what it was given
    (numpy array or DeviceTensor) in the shape of out."""
    out, obj, batch, steps, size, space, ptr = _loss_args(out, obj, sequential)
    if space == DEVICE:
        grad = DeviceTensor(out.shape, out.dtype)
    else:
        grad = np.empty(out.shape, dtype=out.dtype, order="F")
    _check(lib().cattle_hip_loss_d_function(_dtype_code(out.dtype), _loss_kind(kind, negated), ptr(out), space, ptr(obj), space,
                                            _sz(batch), _sz(steps), _sz(size), ctypes.c_double(epsilon),
                                            ctypes.c_double(scale), ptr(grad), space))
    return grad


class Layer(object):
    """Base of the layer mirrors; subclasses create the handle."""

    def __init__(self, handle, dtype, in_shape, out_shape):
        self._h = handle
        self.dtype = np.dtype(dtype)
        self._in_shape = tuple(in_shape)        # per-sample shapes as the caller sees them
        self._out_shape = tuple(out_shape)

    # -- cattle::Layer ------------------------------------------------------------------------
    def get_input_dims(self):
        return self._in_shape

    def get_output_dims(self):
        return self._out_shape

    def is_input_layer(self):
        v = ctypes.c_int()
        _check(lib().cattle_hip_layer_is_input_layer(self._h, ctypes.byref(v)))
        return bool(v.value)

    def set_input_layer(self, flag):
        _check(lib().cattle_hip_layer_set_input_layer(self._h, ctypes.c_int(int(bool(flag)))))

    def empty_cache(self):
        _check(lib().cattle_hip_layer_empty_cache(self._h))

    def get_params(self):
        n = ctypes.c_size_t()
        _check(lib().cattle_hip_layer_num_params(self._h, ctypes.byref(n)))
        return [Parameters(self, i) for i in range(int(n.value))]

    def _clone(self, share):
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_layer_clone(self._h, ctypes.c_int(int(share)), ctypes.byref(h)))
        c = object.__new__(type(self))
        c.__dict__.update(self.__dict__)
        c._h = h
        return c

    def clone(self):
        return self._clone(False)

    def clone_with_shared_params(self):
        return self._clone(True)

    def pass_forward(self, x, training):
        """x: numpy array (host path, returns numpy) or DeviceTensor (device path, returns DeviceTensor)."""
        if isinstance(x, DeviceTensor):
            batch = x.shape[0]
            self._expect(x.shape[1:], self._in_shape, "input")
            out = DeviceTensor((batch,) + self._out_shape, self.dtype)
            _check(lib().cattle_hip_layer_forward(self._h, x.ptr, DEVICE, _sz(batch), ctypes.c_int(int(training)), out.ptr, DEVICE))
            self._keep = (x, out)                 # borrowed by the layer until pass_back
            return out
        x = np.asfortranarray(x, dtype=self.dtype)
        batch = x.shape[0]
        self._expect(x.shape[1:], self._in_shape, "input")
        out = np.empty((batch,) + self._out_shape, dtype=self.dtype, order="F")
        _check(lib().cattle_hip_layer_forward(self._h, ctypes.c_void_p(x.ctypes.data), HOST, _sz(batch),
                                              ctypes.c_int(int(training)), ctypes.c_void_p(out.ctypes.data), HOST))
        return out

    def forward_into(self, x, out, training=True):
        """Device path without allocation: x and out are DeviceTensors owned by the caller."""
        _check(lib().cattle_hip_layer_forward(self._h, x.ptr, DEVICE, _sz(x.shape[0]), ctypes.c_int(int(training)), out.ptr,
                                              DEVICE))

    def backward_into(self, out_grad, in_grad):
        """Device path without allocation; in_grad may be None for an input layer."""
        _check(lib().cattle_hip_layer_backward(self._h, out_grad.ptr, DEVICE, _sz(out_grad.shape[0]),
                                               None if in_grad is None else in_grad.ptr, DEVICE))

    def pass_back(self, out_grad):
        """Returns the input gradient, or None for an input layer (the reference's null tensor)."""
        skip = self.is_input_layer() and not getattr(self, "_always_backprop", False)
        if isinstance(out_grad, DeviceTensor):
            batch = out_grad.shape[0]
            self._expect(out_grad.shape[1:], self._out_shape, "output gradient")
            dx = None if skip else DeviceTensor((batch,) + self._in_shape, self.dtype)
            _check(lib().cattle_hip_layer_backward(self._h, out_grad.ptr, DEVICE, _sz(batch), None if skip else dx.ptr, DEVICE))
            return dx
        g = np.asfortranarray(out_grad, dtype=self.dtype)
        batch = g.shape[0]
        self._expect(g.shape[1:], self._out_shape, "output gradient")
        dx = None if skip else np.empty((batch,) + self._in_shape, dtype=self.dtype, order="F")
        _check(lib().cattle_hip_layer_backward(self._h, ctypes.c_void_p(g.ctypes.data), HOST, _sz(batch),
                                               None if skip else ctypes.c_void_p(dx.ctypes.data), HOST))
        return dx

    @staticmethod
    def _expect(got, want, what):
        if tuple(got) != tuple(want):
            raise ValueError("%s dimensions %s do not match the layer's %s" % (what, tuple(got), tuple(want)))

    def __del__(self):
        try:
            if self._h is not None and self._h.value:
                lib().cattle_hip_layer_destroy(self._h)
        except Exception:
            pass
        self._h = None


def _ext3(dims):
    """Dimensions::extend<3 - Rank>() (core/Dimensions.hpp:63-103): pad with ones to rank 3."""
    dims = tuple(int(d) for d in dims)
    return dims + (1,) * (3 - len(dims))


class ConvKernelLayer(Layer):
    """layer/kernel/ConvKernelLayer.hpp:282-296; rank 1/2 inputs are re-viewed as in :400-417, :494-508."""

    def __init__(self, dtype, input_dims, filters, receptor_height=3, receptor_width=3, vertical_padding=1,
                 horizontal_padding=1, vertical_stride=1, horizontal_stride=1, vertical_dilation=0,
                 horizontal_dilation=0):
        rank = len(input_dims)
        if rank == 1:       # ConvKernelLayer<Scalar,1>: (length) -> receptor (len,1), padding (p,0), stride (s,1)
            receptor_width, horizontal_padding, horizontal_stride, horizontal_dilation = 1, 0, 1, 0
        H, W, C = _ext3(input_dims)
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_conv_create(_dtype_code(dtype), _sz(H), _sz(W), _sz(C), _sz(filters), _sz(receptor_height),
                                            _sz(receptor_width), _sz(vertical_padding), _sz(horizontal_padding),
                                            _sz(vertical_stride), _sz(horizontal_stride), _sz(vertical_dilation),
                                            _sz(horizontal_dilation), ctypes.byref(h)))
        od = (ctypes.c_size_t * 3)()
        _check(lib().cattle_hip_layer_output_dims(h, od))
        OH, OW, F = int(od[0]), int(od[1]), int(od[2])
        # calculate_adjusted_output_dims (:206-217): filters land on the last nominal rank
        out = {3: (OH, OW, F), 2: (OH, OW * F), 1: (OH * F,)}[rank]
        Layer.__init__(self, h, dtype, tuple(input_dims), out)


class TransConvKernelLayer(Layer):
    """layer/kernel/TransConvKernelLayer.hpp:290-304; rank 1/2 inputs are re-viewed as in :404-417, :503-516 and the
    filters land on the last nominal rank of the output (calculate_adjusted_output_dims, :241-251)."""

    def __init__(self, dtype, input_dims, filters, receptor_height=3, receptor_width=3, vertical_padding=1,
                 horizontal_padding=1, vertical_stride=1, horizontal_stride=1, vertical_dilation=0,
                 horizontal_dilation=0):
        rank = len(input_dims)
        if rank == 1:       # TransConvKernelLayer<Scalar,1>(dims, filters, init, receptor_length, padding, stride, dilation)
            receptor_width, horizontal_padding, horizontal_stride, horizontal_dilation = 1, 0, 1, 0
        H, W, C = _ext3(input_dims)
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_transconv_create(_dtype_code(dtype), _sz(H), _sz(W), _sz(C), _sz(filters),
                                                 _sz(receptor_height), _sz(receptor_width), _sz(vertical_padding),
                                                 _sz(horizontal_padding), _sz(vertical_stride), _sz(horizontal_stride),
                                                 _sz(vertical_dilation), _sz(horizontal_dilation), ctypes.byref(h)))
        od = (ctypes.c_size_t * 3)()
        _check(lib().cattle_hip_layer_output_dims(h, od))
        OH, OW, F = int(od[0]), int(od[1]), int(od[2])
        out = {3: (OH, OW, F), 2: (OH, OW * F), 1: (OH * F,)}[rank]
        Layer.__init__(self, h, dtype, tuple(input_dims), out)


class _LstmKernelParameters(object):
    """The weights or the bias of one of the eight kernels of a ConvLSTMNetwork: a block of columns of a fused parameter."""

    def __init__(self, net, kernel, bias, rows, cols):
        self._net, self._kernel, self._bias, self._rows, self._cols = net, kernel, int(bias), rows, cols

    def get_rows(self):
        return self._rows

    def get_cols(self):
        return self._cols

    def are_optimizable(self):
        return True

    def _get(self, fn):
        a = np.empty((self._rows, self._cols), dtype=self._net.dtype, order="F")
        _check(fn(self._net._h, _sz(self._kernel), ctypes.c_int(self._bias), ctypes.c_void_p(a.ctypes.data), HOST))
        return a

    def get_values(self):
        return self._get(lib().cattle_hip_convlstm_get_kernel_values)

    def get_grad(self):
        return self._get(lib().cattle_hip_convlstm_get_kernel_grad)

    def set_values(self, values):
        a = np.asfortranarray(values, dtype=self._net.dtype)
        if a.shape != (self._rows, self._cols):
            raise ValueError("expected a %dx%d matrix" % (self._rows, self._cols))
        _check(lib().cattle_hip_convlstm_set_kernel_values(self._net._h, _sz(self._kernel), ctypes.c_int(self._bias),
                                                           ctypes.c_void_p(a.ctypes.data), HOST))


class ConvLSTMNetwork(Layer):
    """LSTMNeuralNetwork<Scalar,3> over eight ConvKernelLayers with fused gates
    (neural_network/LSTMNeuralNetwork.hpp:27-120, :236-503). activations: forget, write, candidate, state, read.
    output_seq_size_func maps the input sequence length to (output length, output delay) (:60-63)."""

    KERNELS = ("input_forget", "output_forget", "input_write", "output_write", "input_candidate", "output_candidate",
               "input_read", "output_read")

    def __init__(self, dtype, input_dims, hidden_channels, receptor_height=3, receptor_width=3, vertical_padding=1,
                 horizontal_padding=1, vertical_dilation=0, horizontal_dilation=0,
                 activations=("sigmoid", "sigmoid", "tanh", "tanh", "sigmoid"), activation_params=(0, 0, 0, 0, 0),
                 output_seq_size_func=lambda input_seq_length: (input_seq_length, 0), foremost=True, mul_int=False):
        H, W, C = (int(d) for d in input_dims)
        kinds = (ctypes.c_int * 5)(*[ACT[a] for a in activations])
        params = (ctypes.c_double * 5)(*[float(p) for p in activation_params])
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_convlstm_create(_dtype_code(dtype), _sz(H), _sz(W), _sz(C), _sz(hidden_channels),
                                                _sz(receptor_height), _sz(receptor_width), _sz(vertical_padding),
                                                _sz(horizontal_padding), _sz(vertical_dilation), _sz(horizontal_dilation),
                                                kinds, params, ctypes.c_int(int(foremost)), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, (H, W, C), (H, W, int(hidden_channels)))
        self._seq = output_seq_size_func
        self._foremost = bool(foremost)
        self._rv = (receptor_height * receptor_width * C, receptor_height * receptor_width * int(hidden_channels))
        self._hidden = int(hidden_channels)
        self._in_seq_shape = None
        if mul_int:         # the MulInt template argument (neural_network/LSTMNeuralNetwork.hpp:44)
            self.set_multiplicative_integration(True)

    def set_multiplicative_integration(self, enabled):
        _check(lib().cattle_hip_convlstm_set_multiplicative_integration(self._h, ctypes.c_int(int(bool(enabled)))))

    def fused_steps(self):
        """(forward, backward): the time steps of the last propagate / backpropagate whose element-wise part ran inside a
        kernel of the output-side convolutions."""
        f, b = ctypes.c_int(), ctypes.c_int()
        _check(lib().cattle_hip_convlstm_fused_steps(self._h, ctypes.byref(f), ctypes.byref(b)))
        return int(f.value), int(b.value)

    def is_foremost(self):
        return self._foremost

    def kernel_params(self, kernel):
        """(weights, bias) of kernel `kernel` (an index or a name of KERNELS)."""
        k = self.KERNELS.index(kernel) if isinstance(kernel, str) else int(kernel)
        return (_LstmKernelParameters(self, k, False, self._rv[k % 2], self._hidden),
                _LstmKernelParameters(self, k, True, 1, self._hidden))

    def propagate(self, x, training=True):
        """x: (N, T, H, W, C) numpy array or DeviceTensor; returns the same kind, (N, T_out, H, W, hidden)."""
        dev = isinstance(x, DeviceTensor)
        if not dev:
            x = np.asfortranarray(x, dtype=self.dtype)
        self._expect(x.shape[2:], self._in_shape, "input")
        N, T = x.shape[0], x.shape[1]
        out_len, delay = self._seq(T)
        shape = (N, out_len) + self._out_shape
        out = DeviceTensor(shape, self.dtype) if dev else np.empty(shape, dtype=self.dtype, order="F")
        ptr = (lambda t: t.ptr) if dev else (lambda a: ctypes.c_void_p(a.ctypes.data))
        space = DEVICE if dev else HOST
        _check(lib().cattle_hip_convlstm_propagate(self._h, ptr(x), space, _sz(N), _sz(T), _sz(out_len), _sz(delay),
                                                   ctypes.c_int(int(training)), ptr(out), space))
        self._in_seq_shape = tuple(x.shape)
        self._keep = (x, out)
        return out

    def backpropagate(self, out_grad):
        """Returns the input gradient (N, T, H, W, C), or None when the network is foremost."""
        dev = isinstance(out_grad, DeviceTensor)
        if not dev:
            out_grad = np.asfortranarray(out_grad, dtype=self.dtype)
        space = DEVICE if dev else HOST
        ptr = (lambda t: t.ptr) if dev else (lambda a: ctypes.c_void_p(a.ctypes.data))
        if self._foremost:
            dx = None
        elif dev:
            dx = DeviceTensor(self._in_seq_shape, self.dtype)
        else:
            dx = np.empty(self._in_seq_shape, dtype=self.dtype, order="F")
        _check(lib().cattle_hip_convlstm_backpropagate(self._h, ptr(out_grad), space, None if dx is None else ptr(dx), space))
        return dx


class DenseKernelLayer(Layer):
    """layer/kernel/DenseKernelLayer.hpp:61-77; output dims are (output_size, 1, ...) (:68)."""

    def __init__(self, dtype, input_dims, output_size):
        vol = int(np.prod(input_dims))
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_dense_create(_dtype_code(dtype), _sz(vol), _sz(output_size), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, tuple(input_dims), (int(output_size),) + (1,) * (len(input_dims) - 1))


class BatchNormLayer(Layer):
    """layer/BatchNormLayer.hpp:66-101 (per_last_rank=True) and :334-361 (False); default as in :28."""

    def __init__(self, dtype, dims, norm_avg_decay=0.1, epsilon=1e-5, per_last_rank=None):
        if per_last_rank is None:
            per_last_rank = len(dims) == 3
        # the statistics group is the last nominal rank: view it as the channel rank
        dims = tuple(int(d) for d in dims)
        lead = int(np.prod(dims[:-1])) if len(dims) > 1 else 1
        H, W, C = (lead, 1, dims[-1]) if per_last_rank else _ext3(dims)
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_batchnorm_create(_dtype_code(dtype), _sz(H), _sz(W), _sz(C), ctypes.c_int(int(per_last_rank)),
                                                 ctypes.c_double(norm_avg_decay), ctypes.c_double(epsilon), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, dims, dims)

    def stats_initialized(self):
        v = ctypes.c_int()
        _check(lib().cattle_hip_batchnorm_get_stats_initialized(self._h, ctypes.byref(v)))
        return bool(v.value)

    def set_stats_initialized(self, flag):
        _check(lib().cattle_hip_batchnorm_set_stats_initialized(self._h, ctypes.c_int(int(bool(flag)))))


class ActivationLayer(Layer):
    """layer/activation/<Name>ActivationLayer.hpp; kind is a key of ACT."""

    def __init__(self, dtype, kind, dims, param=0.0):
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_activation_create(_dtype_code(dtype), ctypes.c_int(ACT[kind]), _sz(int(np.prod(dims))),
                                                  ctypes.c_double(param), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, tuple(dims), tuple(dims))
        self.kind = kind
        self._always_backprop = kind == "prelu"


def ReLUActivationLayer(dtype, dims):
    return ActivationLayer(dtype, "relu", dims)


def SigmoidActivationLayer(dtype, dims):
    return ActivationLayer(dtype, "sigmoid", dims)


def TanhActivationLayer(dtype, dims):
    return ActivationLayer(dtype, "tanh", dims)


def _dims3(dims):
    return (ctypes.c_size_t * 3)(*_ext3(dims))


class DropoutLayer(Layer):
    """layer/DropoutLayer.hpp:33-96. `seed` keys the generator of the uniform numbers (the reference uses Eigen's global
    one); the mask of training pass q is a function of (seed, q) and the element index."""

    def __init__(self, dtype, dims, dropout_prob, epsilon=1e-5, seed=0):
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_dropout_create(_dtype_code(dtype), _sz(int(np.prod(dims))), ctypes.c_double(dropout_prob),
                                               ctypes.c_double(epsilon), ctypes.c_ulonglong(seed), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, tuple(dims), tuple(dims))


class ReshapeLayer(Layer):
    """layer/ReshapeLayer.hpp:31-90"""

    def __init__(self, dtype, input_dims, output_dims):
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_reshape_create(_dtype_code(dtype), _dims3(input_dims), _dims3(output_dims), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, tuple(input_dims), tuple(output_dims))


class BroadcastLayer(Layer):
    """layer/BroadcastLayer.hpp:31-101"""

    def __init__(self, dtype, input_dims, broadcast):
        if len(broadcast) != len(input_dims):
            raise ValueError("one repetition count per rank")
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_broadcast_create(_dtype_code(dtype), _dims3(input_dims), _dims3(broadcast), ctypes.byref(h)))
        Layer.__init__(self, h, dtype, tuple(input_dims), tuple(int(d) * int(b) for d, b in zip(input_dims, broadcast)))


class _PoolLayer(Layer):
    def __init__(self, kind, dtype, input_dims, receptor_height, receptor_width, vertical_stride, horizontal_stride):
        rank = len(input_dims)
        if rank == 1:       # Max/MeanPoolLayer<Scalar,1>(dims, receptor_length, stride)
            receptor_width, horizontal_stride = 1, 1
        H, W, C = _ext3(input_dims)
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_pool_create(_dtype_code(dtype), ctypes.c_int(kind), _sz(H), _sz(W), _sz(C), _sz(receptor_height),
                                            _sz(receptor_width), _sz(vertical_stride), _sz(horizontal_stride), ctypes.byref(h)))
        od = (ctypes.c_size_t * 3)()
        _check(lib().cattle_hip_layer_output_dims(h, od))
        out = (int(od[0]), int(od[1]), int(od[2]))[:rank]
        Layer.__init__(self, h, dtype, tuple(input_dims), out)


class MaxPoolLayer(_PoolLayer):
    """layer/pool/MaxPoolLayer.hpp:105-108 (defaults 2x2 stride 2)."""

    def __init__(self, dtype, input_dims, receptor_height=2, receptor_width=2, vertical_stride=2, horizontal_stride=2):
        _PoolLayer.__init__(self, POOL_MAX, dtype, input_dims, receptor_height, receptor_width, vertical_stride,
                            horizontal_stride)

    def max_indices(self, batch):
        """The argmax cache, shape (OH*OW, C*batch), as layer/pool/MaxPoolLayer.hpp:58-62 stores it."""
        od = _ext3(self._out_shape)
        a = np.empty((od[0] * od[1], od[2] * batch), dtype=np.uint32)
        _check(lib().cattle_hip_maxpool_indices(self._h, ctypes.c_void_p(a.ctypes.data), HOST))
        return a


class MeanPoolLayer(_PoolLayer):
    """layer/pool/MeanPoolLayer.hpp:62-65."""

    def __init__(self, dtype, input_dims, receptor_height=2, receptor_width=2, vertical_stride=2, horizontal_stride=2):
        _PoolLayer.__init__(self, POOL_MEAN, dtype, input_dims, receptor_height, receptor_width, vertical_stride,
                            horizontal_stride)


class FusedKernelLayer(Layer):
    """A kernel layer and the batch norm / activation / pool layers behind it as one layer (cattle_hip_fused_create): the
    calls FeedforwardNeuralNetwork.hpp:112-141 makes one after another. The members keep their parameters and caches."""

    MODES = {0: "none", 1: "unfused", 2: "act", 3: "pool", 4: "bn"}

    def __init__(self, members):
        members = list(members)
        handles = (ctypes.c_void_p * len(members))(*[m._h for m in members])
        h = ctypes.c_void_p()
        _check(lib().cattle_hip_fused_create(handles, _sz(len(members)), ctypes.byref(h)))
        Layer.__init__(self, h, members[0].dtype, members[0].get_input_dims(), members[-1].get_output_dims())
        self.members = members          # borrowed by the handle: keep them alive

    def last_mode(self):
        v = ctypes.c_int()
        _check(lib().cattle_hip_fused_last_mode(self._h, ctypes.byref(v)))
        return self.MODES[int(v.value)]

    def _clone(self, share):
        c = Layer._clone(self, share)
        c.members = []                  # the clone's handle owns clones of the members
        return c

    def __del__(self):
        Layer.__del__(self)             # the fused handle goes before its members
        self.members = None


def fuse_layers(layers):
    """The layer list of a feed-forward network with every convolutional or dense layer and the batch norm, activation
    and pool layers right behind it (in this order, each optional) replaced by one FusedKernelLayer over them; the other
    layers stay as they are. Calling the result in order equals calling `layers` in order."""
    out, i = [], 0
    while i < len(layers):
        group = [layers[i]]
        if isinstance(layers[i], (ConvKernelLayer, DenseKernelLayer)):
            for cls in (BatchNormLayer, ActivationLayer, _PoolLayer):
                j = i + len(group)
                if j < len(layers) and isinstance(layers[j], cls) and layers[j].dtype == layers[i].dtype:
                    group.append(layers[j])
        if len(group) > 1:
            fused = FusedKernelLayer(group)
            fused.set_input_layer(group[0].is_input_layer())
            out.append(fused)
        else:
            out.append(layers[i])
        i += len(group)
    return out


class Graph(object):
    """A recorded sequence of device-side calls (cattle_hip_graph_*): `with Graph() as g: step()` records what step()
    issues instead of running it, g.launch() runs it. step() must have run once before, use device tensors only and read
    nothing back; the tensors it uses and creates belong to the graph until the graph is destroyed."""

    def __init__(self):
        self._h = None

    def __enter__(self):
        _check(lib().cattle_hip_graph_begin_capture())
        return self

    def __exit__(self, exc_type, exc, tb):
        h = ctypes.c_void_p()
        rc = lib().cattle_hip_graph_end_capture(ctypes.byref(h))
        if exc_type is None:
            _check(rc)
            self._h = h
        elif rc == 0:
            # the body failed: the graph is of no use, and dropping its handle would keep the graph and every pool
            # block of the recording out of circulation for good
            lib().cattle_hip_graph_destroy(h)
        return False

    def launch(self):
        _check(lib().cattle_hip_graph_launch(self._h))

    def destroy(self):
        if self._h is not None:
            _check(lib().cattle_hip_graph_destroy(self._h))
            self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
