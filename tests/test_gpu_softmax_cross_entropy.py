"""GPU parity of the fused softmax -> cross-entropy forward and backward
(lbn_softmax_cross_entropy_fwd_f32, lbn_softmax_cross_entropy_bwd_f32).

The oracle is the composition of the two restatements: cross_entropy_fwd(softmax_fwd(x), truth)
(src/layers/activations/softmax.cpp:43-109 followed by src/layers/loss/cross_entropy.cpp:35-73).
The fused call must also agree with the library's own two calls made one after the other:
y bit for bit where both take the register kernels, the loss within the fp32 tolerance
(the order of its sum differs).  Tolerance: 1e-5 (tests/parity.py), with the float64 leg for
the long sums.
"""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()
    assert torch.cuda.is_available()
    return layers


def rand(rng, h, w, mean=0.0, std=1.0):
    return np.asfortranarray((rng.standard_normal((w, h)) * std + mean).astype(np.float32).T)


def dense_truth(rng, h, w, kind):
    if kind == "one_hot":
        t = np.zeros((h, w), np.float32)
        t[rng.integers(0, h, w), np.arange(w)] = 1.0
    elif kind == "soft":  # a distribution per column, with exact zeros and negative entries (both skipped)
        t = rng.random((h, w)).astype(np.float32)
        t[rng.random((h, w)) < 0.3] = 0.0
        t[rng.random((h, w)) < 0.05] = -0.5
        t /= np.maximum(np.abs(t).sum(axis=0, keepdims=True), 1e-6)
    return np.asfortranarray(t)


def separate(L, x, t, dims, use_labels, ldx=None, ldt=None):
    sm, ce = L.softmax_layer(), L.cross_entropy_layer(dims, use_labels)
    y = sm.forward(L.DeviceMatrix.from_numpy(x, ldim=ldx))
    loss = ce.forward(y, L.DeviceMatrix.from_numpy(t, ldim=ldt))
    return y.to_numpy(), loss.to_numpy()[0]


def fused(L, x, t, dims, use_labels, ldx=None, ldt=None):
    sm, ce = L.softmax_layer(), L.cross_entropy_layer(dims, use_labels)
    y, loss = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x, ldim=ldx),
                                              L.DeviceMatrix.from_numpy(t, ldim=ldt))
    return y.to_numpy(), loss.to_numpy()[0], sm, ce


def oracle(x, t, use_labels):
    y = orc.softmax_fwd(x)
    y64 = orc.softmax_fwd(x.astype(np.float64))
    return y, orc.cross_entropy_fwd(y, t, use_labels), y64, orc.cross_entropy_fwd(y64, t.astype(np.float64), use_labels)


# (h, w, pad): register kernels of every team width; shapes the fused kernel refuses
# (odd heights, unaligned leading dimension, rows past 32768) that run as two kernels
DENSE_SHAPES = [(16, 700, 0), (64, 300, 0), (128, 4100, 0), (1000, 130, 0), (1024, 33, 0), (4096, 40, 0),
                (8192, 9, 0), (20000, 5, 0), (32768, 3, 0), (512, 7, 64),
                (10, 300, 0), (1001, 9, 0), (130, 3, 3), (50257, 6, 0), (65536, 3, 0), (1, 5, 0), (4, 1, 0)]


@pytest.mark.parametrize("h,w,pad", DENSE_SHAPES)
@pytest.mark.parametrize("kind", ["one_hot", "soft"])
def test_dense(L, h, w, pad, kind):
    rng = np.random.default_rng(h * 131 + w)
    x, t = rand(rng, h, w, 0, 3), dense_truth(rng, h, w, kind)
    ld = h + pad if pad else None
    y, loss, sm, ce = fused(L, x, t, (h,), False, ld, ld)
    y_ref, loss_ref, y64, loss64 = oracle(x, t, False)
    check(f"softmax_ce dense {kind} {h}x{w} y", y, y_ref, y64)
    check(f"softmax_ce dense {kind} {h}x{w} loss", loss, loss_ref, loss64)
    y2, loss2 = separate(L, x, t, (h,), False, ld, ld)
    if h * w * 4 < (48 << 20):
        assert np.array_equal(y, y2), "fused y differs from lbn_softmax_fwd_f32's"
    check(f"softmax_ce dense {kind} {h}x{w} loss vs two calls", loss, loss2, loss64)


@pytest.mark.parametrize("classes,spatial,w", [(10, 1, 300), (1000, 1, 64), (1024, 1, 33), (50257, 1, 6), (32768, 1, 3),
                                               (4, 64, 9), (21, 100, 7)])
def test_labels(L, classes, spatial, w):
    """spatial == 1 takes the fused kernel (when the row does); larger spatial sizes run as two kernels."""
    rng = np.random.default_rng(classes + spatial)
    h = classes * spatial
    x = rand(rng, h, w, 0, 3)
    t = np.asfortranarray(rng.integers(0, classes, (spatial, w)).astype(np.float32))
    t[0, 0] = -1.0           # no class: contributes nothing
    if w > 1:
        t[0, 1] = classes    # past the last class: contributes nothing
    y, loss, _, _ = fused(L, x, t, (classes, spatial), True)
    y_ref, loss_ref, y64, loss64 = oracle(x, t, True)
    check(f"softmax_ce labels {classes}x{spatial}x{w} y", y, y_ref, y64)
    check(f"softmax_ce labels {classes}x{spatial}x{w} loss", loss, loss_ref, loss64)
    _, loss2 = separate(L, x, t, (classes, spatial), True)
    check(f"softmax_ce labels {classes}x{spatial}x{w} loss vs two calls", loss, loss2, loss64)


def test_flushed_entry_under_positive_truth_is_infinite(L):
    """An output flushed to zero (softmax.cpp:98-105) under xhat > 0 gives log(0): the loss is
    +inf, as it is when the two layers run one after the other."""
    h, w = 1024, 4
    x = np.zeros((h, w), np.float32, order="F")
    x[0, :] = 200.0     # every other entry underflows
    t = np.zeros((h, w), np.float32, order="F")
    t[0, 0] = 1.0       # finite: picks the surviving entry
    t[5, 1] = 1.0       # flushed entry
    t[5, 2] = -1.0      # negative: skipped
    y, loss, _, _ = fused(L, x, t, (h,), False)
    y_ref, loss_ref, _, _ = oracle(x, t, False)
    assert np.array_equal(np.isinf(loss), np.isinf(loss_ref))
    assert np.isinf(loss[1]) and loss[1] > 0 and loss[0] == 0.0 and loss[2] == 0.0 and loss[3] == 0.0
    check("softmax_ce flushed y", y, y_ref)
    tl = np.asfortranarray(np.array([[0.0, 5.0, 0.0, 7.0]], np.float32))
    _, loss, _, _ = fused(L, x, tl, (h, 1), True)
    assert loss[0] == 0.0 and np.isinf(loss[1]) and loss[2] == 0.0 and np.isinf(loss[3])


def test_backward_after_fused_forward(L):
    """Both layers' members are bound as their own forward binds them: each backward runs unchanged."""
    rng = np.random.default_rng(5)
    h, w = 1000, 48
    x, t = rand(rng, h, w, 0, 2), dense_truth(rng, h, w, "soft")
    y, loss, sm, ce = fused(L, x, t, (h,), False)
    g = rng.standard_normal(w).astype(np.float32)
    dpred, dtruth = ce.backward(L.DeviceMatrix.from_numpy(g.reshape(1, w)))
    dx = sm.backward(dpred).to_numpy()
    dp_ref, dt_ref = orc.cross_entropy_bwd(y, t, g)
    check("softmax_ce bwd dprediction", dpred.to_numpy(), dp_ref)
    check("softmax_ce bwd dtruth", dtruth.to_numpy(), dt_ref)
    check("softmax_ce bwd dx", dx, orc.softmax_bwd(y, dp_ref))


@pytest.mark.parametrize("h,w,pad", DENSE_SHAPES)
@pytest.mark.parametrize("want_dtruth", [False, True])
def test_backward_dense(L, h, w, pad, want_dtruth):
    """Oracle: softmax_bwd(y, cross_entropy_bwd(y, truth, dloss).dprediction), the composition of
    the two restatements (cross_entropy.cpp:75-120, openmp/softmax.hpp:119-181); also against the
    library's own two calls."""
    rng = np.random.default_rng(h * 17 + w)
    x, t = rand(rng, h, w, 0, 2), dense_truth(rng, h, w, "soft")
    g = rng.standard_normal(w).astype(np.float32)
    ld = h + pad if pad else None
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((h,))
    y, _ = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x, ldim=ld),
                                           L.DeviceMatrix.from_numpy(t, ldim=ld))
    yh = y.to_numpy()
    dx = L.softmax_cross_entropy_backward(sm, ce, L.DeviceMatrix.from_numpy(g.reshape(1, w)), want_dtruth)
    dp_ref, dt_ref = orc.cross_entropy_bwd(yh, t, g)
    y64 = yh.astype(np.float64)
    dp64, dt64 = orc.cross_entropy_bwd(np.asfortranarray(y64), np.asfortranarray(t.astype(np.float64)), g.astype(np.float64))
    check(f"softmax_ce bwd dense {h}x{w} dx", dx.to_numpy(), orc.softmax_bwd(yh, dp_ref),
          orc.softmax_bwd(np.asfortranarray(y64), dp64))
    if want_dtruth:
        check(f"softmax_ce bwd dense {h}x{w} dtruth", ce.error_signals[1].to_numpy(), dt_ref, dt64)
    else:
        assert ce.error_signals[1] is None
    # the two calls one after the other, on the same y
    sm2, ce2 = L.softmax_layer(), L.cross_entropy_layer((h,))
    L.softmax_cross_entropy_forward(sm2, ce2, L.DeviceMatrix.from_numpy(x, ldim=ld), L.DeviceMatrix.from_numpy(t, ldim=ld))
    dpred, _ = ce2.backward(L.DeviceMatrix.from_numpy(g.reshape(1, w)))
    dx2 = sm2.backward(dpred).to_numpy()
    check(f"softmax_ce bwd dense {h}x{w} dx vs two calls", dx.to_numpy(), dx2, orc.softmax_bwd(np.asfortranarray(y64), dp64))


@pytest.mark.parametrize("classes,spatial,w", [(10, 1, 300), (1000, 1, 64), (1024, 1, 33), (50257, 1, 6), (32768, 1, 3),
                                               (4, 64, 9), (21, 100, 7)])
def test_backward_labels(L, classes, spatial, w):
    rng = np.random.default_rng(classes * 3 + spatial)
    h = classes * spatial
    x = rand(rng, h, w, 0, 2)
    t = np.asfortranarray(rng.integers(0, classes, (spatial, w)).astype(np.float32))
    t[0, 0] = -1.0
    g = rng.standard_normal(w).astype(np.float32)
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((classes, spatial), True)
    y, _ = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x), L.DeviceMatrix.from_numpy(t))
    yh = y.to_numpy()
    dx = L.softmax_cross_entropy_backward(sm, ce, L.DeviceMatrix.from_numpy(g.reshape(1, w)))
    dp_ref, _ = orc.cross_entropy_bwd(yh, t, g, True)
    y64 = np.asfortranarray(yh.astype(np.float64))
    dp64, _ = orc.cross_entropy_bwd(y64, np.asfortranarray(t.astype(np.float64)), g.astype(np.float64), True)
    check(f"softmax_ce bwd labels {classes}x{spatial}x{w} dx", dx.to_numpy(), orc.softmax_bwd(yh, dp_ref),
          orc.softmax_bwd(y64, dp64))


def test_backward_flushed_entry_gives_the_same_nan(L):
    """y flushed to zero under xhat > 0: the gradient with respect to the prediction is -inf there
    and the softmax backward turns the column into NaN, fused or not."""
    h, w = 1024, 3
    x = np.zeros((h, w), np.float32, order="F")
    x[0, :] = 200.0
    t = np.zeros((h, w), np.float32, order="F")
    t[0, 0] = 1.0
    t[5, 1] = 1.0       # flushed entry under a positive xhat
    g = np.ones(w, np.float32)
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((h,))
    y, _ = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x), L.DeviceMatrix.from_numpy(t))
    yh = y.to_numpy()
    dx = L.softmax_cross_entropy_backward(sm, ce, L.DeviceMatrix.from_numpy(g.reshape(1, w))).to_numpy()
    with np.errstate(all="ignore"):
        ref = orc.softmax_bwd(yh, orc.cross_entropy_bwd(yh, t, g)[0])
    assert np.array_equal(np.isnan(dx), np.isnan(ref))
    assert np.isnan(dx[:, 1]).all() and np.isfinite(dx[:, 0]).all() and np.all(dx[:, 2] == 0)
    ok = ~np.isnan(ref)
    check("softmax_ce bwd flushed finite part", np.where(ok, dx, 0), np.where(ok, ref, 0))


def test_empty_and_bad_arguments(L):
    capi = L.capi
    null = capi.vp(None)
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    fn = capi.lib().lbn_softmax_cross_entropy_fwd_f32
    loss = torch.full((5,), 7.0, device="cuda")
    assert fn(st, 0, 5, 0, 1, null, 1, null, 1, null, 1, capi.vp(loss.data_ptr()), 1, null, 0) == 0
    assert torch.all(loss == 0).item()  # empty columns: the loss is written, and is 0
    assert fn(st, 0, 5, 0, 1, null, 1, null, 1, null, 1, null, 1, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert fn(st, 8, 0, 0, 1, null, 8, null, 8, null, 8, null, 1, null, 0) == 0
    assert fn(st, -1, 5, 0, 1, null, 1, null, 1, null, 1, null, 1, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert fn(st, 8, 2, 0, 1, null, 8, null, 8, null, 8, null, 1, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    buf = torch.zeros(64, device="cuda")
    p = capi.vp(buf.data_ptr())
    assert fn(st, 8, 2, 0, 1, p, 4, p, 8, p, 8, p, 1, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT  # ldx < height
