"""ctypes binding of the CPU oracle (oracle/lbann_cpu_oracle.cpp).

TEST INFRASTRUCTURE ONLY.  This module is the checker for the HIP kernels and
the CPU baseline leg of the benchmark; the product package never imports it.

All matrices are NumPy arrays in Fortran (column-major) order with shape
(height, width): element (r, c) lives at buf[r + c*ld], one column per sample,
the layout of LBANN's local El::Matrix.  dtype selects the `_f32` or `_f64`
instantiation of the restated reference code.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblbann_cpu_oracle.so")
_lib = None

_i64 = ctypes.c_int64
_vp = ctypes.c_void_p


def lib():
    """Load the oracle library, compiling it first if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _build
            _build.build(force=True)
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_max_threads.restype = ctypes.c_int
    return _lib


def max_threads() -> int:
    return int(lib().orc_max_threads())


def _suffix(a):
    if a.dtype == np.float32:
        return "f32", ctypes.c_float
    if a.dtype == np.float64:
        return "f64", ctypes.c_double
    raise TypeError(f"oracle supports float32/float64, got {a.dtype}")


def _mat(a):
    """(pointer, leading dimension) of a column-major 2-D array."""
    assert a.ndim == 2 and (a.strides[0] == a.itemsize or a.shape[0] <= 1), "matrix must be column-major"
    ld = a.strides[1] // a.itemsize if a.shape[1] > 1 else max(a.shape[0], 1)
    assert ld >= a.shape[0]
    return _vp(a.ctypes.data), _i64(ld)


def _vec(a):
    if a is None:
        return _vp(None)
    assert a.flags["C_CONTIGUOUS"] or a.flags["F_CONTIGUOUS"]
    return _vp(a.ctypes.data)


def fmat(h, w, dtype):
    return np.empty((h, w), dtype=dtype, order="F")


# ------------------------------------------------------------------ layer norm
def layer_norm_fwd(x, G, n, stride, eps, gamma=None, beta=None):
    """Returns (y, stats) with stats (2G x w): rows [0,G) mean, [G,2G) variance."""
    suf, cf = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    stats = fmat(2 * G, w, x.dtype)
    fn = getattr(lib(), f"orc_layer_norm_fwd_{suf}")
    fn(_i64(G), _i64(n), _i64(stride), _i64(w), cf(eps), *_mat(x), *_mat(y),
       *_mat(stats), _vec(gamma), _vec(beta))
    return y, stats


def layer_norm_bwd(x, dy, stats, G, n, stride, eps, gamma=None, want_dgamma=False,
                   want_dbeta=False):
    """Returns (dx, stats_grad, dgamma|None, dbeta|None)."""
    suf, cf = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    sgrad = np.zeros((2 * G, w), dtype=x.dtype, order="F")
    dgamma = np.empty(n, dtype=x.dtype) if want_dgamma else None
    dbeta = np.empty(n, dtype=x.dtype) if want_dbeta else None
    fn = getattr(lib(), f"orc_layer_norm_bwd_{suf}")
    fn(_i64(G), _i64(n), _i64(stride), _i64(w), _i64(h), cf(eps), *_mat(x), *_mat(dy),
       *_mat(dx), *_mat(stats), *_mat(sgrad), _vec(gamma), _vec(dgamma), _vec(dbeta))
    return dx, sgrad, dgamma, dbeta


# ------------------------------------------------------------------ batch norm
def batch_norm_fwd(x, C, cs, eps, decay, gamma, beta, running_mean, running_var,
                   bessel=True, training=True):
    """Returns (y, mean, var); running_mean/var are updated in place when training."""
    suf, cf = _suffix(x)
    h, w = x.shape
    assert h == C * cs
    y = fmat(h, w, x.dtype)
    mean = np.zeros(C, dtype=x.dtype)
    var = np.zeros(C, dtype=x.dtype)
    fn = getattr(lib(), f"orc_batch_norm_fwd_{suf}")
    fn(_i64(C), _i64(cs), _i64(w), ctypes.c_int(int(bessel)), cf(eps), cf(decay),
       ctypes.c_int(int(training)), *_mat(x), *_mat(y), _vec(mean), _vec(var),
       _vec(gamma), _vec(beta), _vec(running_mean), _vec(running_var))
    return y, mean, var


def batch_norm_bwd(x, dy, C, cs, eps, mean, var, gamma, running_mean=None,
                   running_var=None, bessel=True, training=True):
    """Returns (dx, dgamma, dbeta, dmean, dvar)."""
    suf, cf = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    dgamma = np.empty(C, dtype=x.dtype)
    dbeta = np.empty(C, dtype=x.dtype)
    dmean = np.empty(C, dtype=x.dtype)
    dvar = np.empty(C, dtype=x.dtype)
    fn = getattr(lib(), f"orc_batch_norm_bwd_{suf}")
    fn(_i64(C), _i64(cs), _i64(w), ctypes.c_int(int(bessel)), cf(eps),
       ctypes.c_int(int(training)), *_mat(x), *_mat(dy), *_mat(dx), _vec(mean), _vec(var),
       _vec(running_mean), _vec(running_var), _vec(gamma), _vec(dgamma), _vec(dbeta),
       _vec(dmean), _vec(dvar))
    return dx, dgamma, dbeta, dmean, dvar


# --------------------------------------------------------- softmax / log-softmax
def _unary(name, x):
    suf, _ = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    getattr(lib(), f"orc_{name}_fwd_{suf}")(_i64(h), _i64(w), *_mat(x), *_mat(y))
    return y


def _unary_bwd(name, y, dy):
    suf, _ = _suffix(y)
    h, w = y.shape
    dx = fmat(h, w, y.dtype)
    getattr(lib(), f"orc_{name}_bwd_{suf}")(_i64(h), _i64(w), *_mat(y), *_mat(dy), *_mat(dx))
    return dx


def softmax_fwd(x):
    return _unary("softmax", x)


def softmax_bwd(y, dy):
    return _unary_bwd("softmax", y, dy)


def log_softmax_fwd(x):
    return _unary("log_softmax", x)


def log_softmax_bwd(y, dy):
    return _unary_bwd("log_softmax", y, dy)


# --------------------------------------------------------- channelwise softmax
def channelwise_softmax_fwd(x, C, cs, stride):
    suf, _ = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    getattr(lib(), f"orc_channelwise_softmax_fwd_{suf}")(
        _i64(C), _i64(cs), _i64(stride), _i64(w), *_mat(x), *_mat(y))
    return y


def channelwise_softmax_bwd(y, dy, C, cs, stride):
    suf, _ = _suffix(y)
    h, w = y.shape
    dx = fmat(h, w, y.dtype)
    getattr(lib(), f"orc_channelwise_softmax_bwd_{suf}")(
        _i64(C), _i64(cs), _i64(stride), _i64(w), *_mat(y), *_mat(dy), *_mat(dx))
    return dx


# --------------------------------------------------------------- instance norm
def instance_norm_fwd(x, C, cs, eps):
    """Returns (y, sums) with sums (2C x w): rows [0,C) sum(x), [C,2C) sum(x^2) per sample."""
    suf, cf = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    sums = np.zeros((2 * C, w), dtype=x.dtype, order="F")
    getattr(lib(), f"orc_instance_norm_fwd_{suf}")(
        _i64(C), _i64(cs), _i64(w), cf(eps), *_mat(x), *_mat(y), *_mat(sums))
    return y, sums


def instance_norm_bwd(x, dy, sums, C, cs, eps):
    suf, cf = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    getattr(lib(), f"orc_instance_norm_bwd_{suf}")(
        _i64(C), _i64(cs), _i64(w), cf(eps), *_mat(x), *_mat(dy), *_mat(dx), *_mat(sums))
    return dx


# ------------------------------------------------------- entry-wise batch norm
def entrywise_batch_norm_fwd(x, decay, eps, running_mean, running_var, training=True):
    """Returns (y, stats) with stats (h x 2): column 0 mean, column 1 variance (Bessel
    corrected) of every entry over the mini-batch; running_mean/var are updated in place
    when training and the batch has more than one sample."""
    suf, cf = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    stats = np.zeros((h, 2), dtype=x.dtype, order="F")
    assert running_mean.dtype == x.dtype and running_var.dtype == x.dtype
    getattr(lib(), f"orc_entrywise_batch_norm_fwd_{suf}")(
        _i64(h), _i64(w), cf(decay), cf(eps), ctypes.c_int(int(training)), *_mat(x), *_mat(y),
        *_mat(stats), _vec(running_mean), _vec(running_var))
    return y, stats


def entrywise_batch_norm_bwd(x, dy, stats, eps, running_var=None, training=True):
    """Returns (dx, stats_grad) with stats_grad (h x 2): dL/dmean, dL/dvar."""
    suf, cf = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    sgrad = np.zeros((h, 2), dtype=x.dtype, order="F")
    getattr(lib(), f"orc_entrywise_batch_norm_bwd_{suf}")(
        _i64(h), _i64(w), cf(eps), ctypes.c_int(int(training)), *_mat(x), *_mat(dy), *_mat(dx),
        *_mat(stats), *_mat(sgrad), _vec(running_var))
    return dx, sgrad


# --------------------------------------------------------------- cross entropy
def cross_entropy_fwd(x, truth, use_labels=False):
    """Returns the (w,) loss.  With use_labels, truth is (spatial x w) class indices stored
    as floating point and x is (classes*spatial x w)."""
    suf, _ = _suffix(x)
    h, w = x.shape
    spatial = truth.shape[0] if use_labels else 1
    loss = np.zeros(w, dtype=x.dtype)
    getattr(lib(), f"orc_cross_entropy_fwd_{suf}")(
        _i64(h), _i64(w), ctypes.c_int(int(use_labels)), _i64(spatial), *_mat(x), *_mat(truth), _vec(loss))
    return loss


def cross_entropy_bwd(x, truth, dy, use_labels=False):
    """dy is the (w,) gradient w.r.t. the loss.  Returns (dx, dtruth); dtruth is None with
    use_labels (the reference leaves it untouched)."""
    suf, _ = _suffix(x)
    h, w = x.shape
    spatial = truth.shape[0] if use_labels else 1
    dx = fmat(h, w, x.dtype)
    dtruth = fmat(h, w, x.dtype)
    dy = np.ascontiguousarray(dy, dtype=x.dtype)
    getattr(lib(), f"orc_cross_entropy_bwd_{suf}")(
        _i64(h), _i64(w), ctypes.c_int(int(use_labels)), _i64(spatial), *_mat(x), *_mat(truth), _vec(dy),
        *_mat(dx), *_mat(dtruth))
    return dx, (None if use_labels else dtruth)


# ------------------------------------------------------------ scale/bias layers
def entrywise_scale_bias_fwd(x, weights):
    """weights is (h x 2): column 0 scale, column 1 bias."""
    suf, _ = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    getattr(lib(), f"orc_entrywise_scale_bias_fwd_{suf}")(_i64(h), _i64(w), *_mat(x), *_mat(y), *_mat(weights))
    return y


def entrywise_scale_bias_bwd(x, dy, weights):
    """Returns (dx, weights_grad) with weights_grad (h x 2)."""
    suf, _ = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    wgrad = np.zeros((h, 2), dtype=x.dtype, order="F")
    getattr(lib(), f"orc_entrywise_scale_bias_bwd_{suf}")(
        _i64(h), _i64(w), *_mat(x), *_mat(dy), *_mat(dx), *_mat(weights), *_mat(wgrad))
    return dx, wgrad


def channelwise_scale_bias_fwd(x, weights, C, cs):
    """weights is (C x 2): column 0 scale, column 1 bias."""
    suf, _ = _suffix(x)
    h, w = x.shape
    y = fmat(h, w, x.dtype)
    getattr(lib(), f"orc_channelwise_scale_bias_fwd_{suf}")(
        _i64(C), _i64(cs), _i64(w), *_mat(x), *_mat(y), *_mat(weights))
    return y


def channelwise_scale_bias_bwd(x, dy, weights, C, cs):
    """Returns (dx, weights_grad) with weights_grad (C x 2)."""
    suf, _ = _suffix(x)
    h, w = x.shape
    dx = fmat(h, w, x.dtype)
    wgrad = np.zeros((C, 2), dtype=x.dtype, order="F")
    getattr(lib(), f"orc_channelwise_scale_bias_bwd_{suf}")(
        _i64(C), _i64(cs), _i64(w), *_mat(x), *_mat(dy), *_mat(dx), *_mat(weights), *_mat(wgrad))
    return dx, wgrad


def gradient_sink(gradient, contribution, buf_scale, alpha):
    """gradient = buf_scale * gradient + alpha * contribution as Scale + Axpy; returns the new gradient."""
    suf, cf = _suffix(contribution)
    h, w = contribution.shape
    g = np.array(gradient, dtype=contribution.dtype, order="F", copy=True)
    assert g.shape == (h, w)
    getattr(lib(), f"orc_gradient_sink_{suf}")(
        _i64(h), _i64(w), cf(buf_scale), cf(alpha), *_mat(contribution), *_mat(g))
    return g
