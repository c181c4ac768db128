"""Pins the CPU oracle (oracle/lbann_cpu_oracle.cpp) before anything is compared with it.

Each oracle function is checked against something that does not share its code:
the float64 closed forms and tolerances of the reference's own layer tests
(tests/golden), torch's library routines and autograd in float64, central finite
differences, and invariants.  The checks are chosen so that a dropped term, a
wrong sign, a wrong divisor (n vs n-1), a transposed operand or a misplaced
epsilon fails at least one of them.
"""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import rel_err

F32_EPS = np.finfo(np.float32).eps


def F(a, dtype=None):
    """Column-major copy (samples become columns): input is (samples, features)."""
    a = np.asarray(a)
    return np.asfortranarray(a.T.astype(dtype or a.dtype))


def metric(y_cols):
    y = np.asarray(y_cols, dtype=np.float64)
    return float(np.mean(np.sum(y * y, axis=0)))


# =============================================================== golden: forward
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-12)])
def test_layer_norm_golden(golden, dt, tol):
    x = F(golden["ln_x"], dt)
    y, stats = orc.layer_norm_fwd(x, 1, 31, 31, 1e-5)
    assert rel_err(y.T, golden["ln_y"]) < tol
    # the reference's own acceptance band on the L2Norm2 metric
    val = float(golden["ln_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS
    xd = golden["ln_x"].astype(np.float64)
    assert rel_err(stats[0], xd.mean(axis=1)) < 10 * tol
    assert rel_err(stats[1], xd.var(axis=1)) < 10 * tol


def test_layer_norm_affine_golden(golden):
    x = F(golden["lna_x"])
    g, b = golden["lna_scale"], golden["lna_bias"]
    y, _ = orc.layer_norm_fwd(x, 1, 31, 31, 1e-5, g, b)
    assert rel_err(y.T, golden["lna_y_exact"]) < 3e-6
    # the tolerance the reference test states: mean squared error <= 1e-8
    assert np.mean((y.T - golden["lna_y_test_scaled_bias"]) ** 2) <= 1e-8
    y, _ = orc.layer_norm_fwd(x, 1, 31, 31, 1e-5, g, None)
    assert np.mean((y.T - golden["lna_y_test_scaled"]) ** 2) <= 1e-8
    y, _ = orc.layer_norm_fwd(x, 1, 31, 31, 1e-5, None, None)
    assert np.mean((y.T - golden["lna_y_test_plain"]) ** 2) <= 1e-8
    # default weights (scale 1, bias 0) equal the plain layer
    y1, _ = orc.layer_norm_fwd(x, 1, 31, 31, 1e-5, np.ones(31, np.float32), np.zeros(31, np.float32))
    assert np.array_equal(y, y1)


@pytest.mark.parametrize("start_dim,G,n", [(-1, 62, 5), (1, 31, 10), (0, 1, 310)])
def test_layer_norm_multidim_golden(golden, start_dim, G, n):
    xs = golden["lnm_x"]
    x = F(xs.reshape(31, -1))
    y, _ = orc.layer_norm_fwd(x, G, n, n, 1e-5)
    assert np.mean((y.T - golden[f"lnm_y_test_sd{start_dim}"].reshape(31, -1)) ** 2) <= 1e-7
    # fp32 E[x^2]-mean^2 on 5 uniform draws cancels a few digits: the reference's own noise
    assert rel_err(y.T, golden[f"lnm_y_exact_sd{start_dim}"].reshape(31, -1)) < 1e-4
    yd, _ = orc.layer_norm_fwd(F(xs.reshape(31, -1), np.float64), G, n, n, 1e-5)
    assert rel_err(yd.T, golden[f"lnm_y_exact_sd{start_dim}"].reshape(31, -1)) < 1e-11


@pytest.mark.parametrize("tag,rows", [("mb14", 14), ("all29", 29)])
@pytest.mark.parametrize("bessel", [0, 1])
def test_batch_norm_golden(golden, tag, rows, bessel):
    xs = golden["bn_x"][:rows]
    for dt, tol in ((np.float32, 3e-6), (np.float64, 1e-12)):
        x = F(xs, dt)
        C, cs = 7, 15
        gamma, beta = np.ones(C, dt), np.zeros(C, dt)
        rm, rv = np.zeros(C, dt), np.ones(C, dt)
        y, mean, var = orc.batch_norm_fwd(x, C, cs, 1e-5, 0.9, gamma, beta, rm, rv, bessel=bool(bessel))
        assert rel_err(y.T, golden[f"bn_{tag}_b{bessel}_y"]) < tol
        assert rel_err(mean, golden[f"bn_{tag}_b{bessel}_mean"]) < tol
        assert rel_err(var, golden[f"bn_{tag}_b{bessel}_var"]) < tol
        # running statistics: one exponential-moving-average step from (0, 1)
        assert rel_err(rm, 0.1 * golden[f"bn_{tag}_b{bessel}_mean"]) < 10 * tol
        assert rel_err(rv, 0.9 + 0.1 * golden[f"bn_{tag}_b{bessel}_var"]) < tol


@pytest.mark.parametrize("dt,tol", [(np.float32, 1e-6), (np.float64, 1e-13)])
def test_softmax_golden(golden, dt, tol):
    y = orc.softmax_fwd(F(golden["sm_x"], dt))
    assert rel_err(y.T, golden["sm_y"]) < tol
    val = float(golden["sm_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS
    assert np.allclose(y.sum(axis=0), 1.0, atol=10 * tol)


@pytest.mark.parametrize("dt,tol", [(np.float32, 1e-6), (np.float64, 1e-13)])
def test_log_softmax_golden(golden, dt, tol):
    y = orc.log_softmax_fwd(F(golden["lsm_x"], dt))
    assert rel_err(y.T, golden["lsm_y"]) < tol
    val = float(golden["lsm_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS
    assert np.allclose(np.exp(y.astype(np.float64)).sum(axis=0), 1.0, atol=20 * tol)


@pytest.mark.parametrize("tag,C,cs", [("default", 5, 14), ("lastdim", 10, 7)])
def test_channelwise_softmax_golden(golden, tag, C, cs):
    for dt, tol in ((np.float32, 1e-6), (np.float64, 1e-13)):
        x = F(golden["cws_x"], dt)
        y = orc.channelwise_softmax_fwd(x, C, cs, cs)
        assert rel_err(y.T, golden[f"cws_y_{tag}"]) < tol
        val = float(golden[f"cws_metric_{tag}"])
        assert abs(metric(y) - val) <= 8 * val * F32_EPS
        # same numbers as a plain softmax over the (cs, C*w) reshaping
        plain = orc.softmax_fwd(np.asfortranarray(x.reshape(cs, -1, order="F")))
        assert rel_err(y.reshape(cs, -1, order="F"), plain) < 4 * tol


# ============================================================ library routines
def test_layer_norm_matches_torch():
    rng = np.random.default_rng(1)
    xs = rng.normal(1.5, 2.0, size=(6, 4, 10))
    g, b = rng.normal(1, 0.3, size=10), rng.normal(0, 0.3, size=10)
    # start_dim=-1: normalise the trailing 10 entries, 4 groups per sample
    y, stats = orc.layer_norm_fwd(F(xs.reshape(6, -1)), 4, 10, 10, 1e-5, g, b)
    t = torch.nn.functional.layer_norm(torch.tensor(xs), (10,), torch.tensor(g), torch.tensor(b), 1e-5)
    assert rel_err(y.T.reshape(6, 4, 10), t.numpy()) < 1e-12
    assert rel_err(stats[:4].T, xs.mean(axis=2)) < 1e-12
    assert rel_err(stats[4:].T, xs.var(axis=2)) < 1e-11


def test_batch_norm_matches_torch_without_bessel():
    rng = np.random.default_rng(2)
    N, C, H, W = 5, 3, 4, 6
    xs = rng.normal(2.0, 3.0, size=(N, C, H, W))
    g, b = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.1, C)
    rm, rv = np.zeros(C), np.ones(C)
    y, mean, var = orc.batch_norm_fwd(F(xs.reshape(N, -1)), C, H * W, 1e-5, 0.9, g, b, rm, rv, bessel=False)
    trm, trv = torch.zeros(C, dtype=torch.float64), torch.ones(C, dtype=torch.float64)
    t = torch.nn.functional.batch_norm(torch.tensor(xs), trm, trv, torch.tensor(g), torch.tensor(b),
                                       training=True, momentum=0.1, eps=1e-5)
    assert rel_err(y.T.reshape(xs.shape), t.numpy()) < 1e-12
    assert rel_err(rm, trm.numpy()) < 1e-12
    # torch's running variance always carries n/(n-1); the layer's follows its own flag
    n = N * H * W
    assert rel_err(rv, 0.9 + 0.1 * xs.var(axis=(0, 2, 3))) < 1e-12
    _, _, var_b = orc.batch_norm_fwd(F(xs.reshape(N, -1)), C, H * W, 1e-5, 0.9, g, b, rm.copy(), rv.copy(), bessel=True)
    assert rel_err(var_b, xs.var(axis=(0, 2, 3)) * n / (n - 1)) < 1e-12


def test_batch_norm_inference_uses_running_stats():
    rng = np.random.default_rng(3)
    xs = rng.normal(size=(4, 2 * 5))
    g, b = rng.uniform(0.5, 1.5, 2), rng.normal(0, 0.1, 2)
    rm, rv = rng.normal(size=2), rng.uniform(0.5, 2, 2)
    rm0, rv0 = rm.copy(), rv.copy()
    y, _, _ = orc.batch_norm_fwd(F(xs), 2, 5, 1e-5, 0.9, g, b, rm, rv, training=False)
    assert np.array_equal(rm, rm0) and np.array_equal(rv, rv0)
    exp = (xs.reshape(4, 2, 5) - rm0[None, :, None]) / np.sqrt(rv0[None, :, None] + 1e-5) * g[None, :, None] + b[None, :, None]
    assert rel_err(y.T.reshape(4, 2, 5), exp) < 1e-13


def test_batch_norm_variance_floor_and_tiny_batches():
    # constant channel: variance 0 is raised to eps, then eps is added again
    x = np.full((6, 1), 3.0, dtype=np.float64, order="F")
    g, b = np.array([2.0]), np.array([0.5])
    rm, rv = np.zeros(1), np.ones(1)
    y, mean, var = orc.batch_norm_fwd(x, 1, 6, 1e-3, 0.9, g, b, rm, rv)
    assert var[0] == 1e-3 and mean[0] == 3.0
    assert np.allclose(y, 0.5)
    # a single value per channel: variance is set to one, running stats untouched
    x = np.array([[4.0], [7.0]], order="F")
    rm, rv = np.zeros(2), np.ones(2)
    y, mean, var = orc.batch_norm_fwd(x, 2, 1, 1e-5, 0.9, np.ones(2), np.zeros(2), rm, rv)
    assert np.array_equal(var, [1.0, 1.0]) and np.array_equal(mean, [4.0, 7.0])
    assert np.array_equal(rm, [0, 0]) and np.array_equal(rv, [1, 1])
    assert np.allclose(y, 0)
    dx, *_ = orc.batch_norm_bwd(x, np.ones_like(x), 2, 1, 1e-5, mean, var, np.ones(2))
    assert np.array_equal(dx, np.zeros_like(x))


def test_layer_norm_single_entry_groups():
    x = F(np.arange(6, dtype=np.float64).reshape(2, 3))
    y, stats = orc.layer_norm_fwd(x, 3, 1, 1, 1e-5)
    assert np.array_equal(stats[:3], x) and np.all(stats[3:] == 1.0) and np.all(y == 0)
    dx, *_ = orc.layer_norm_bwd(x, np.ones_like(x), stats, 3, 1, 1, 1e-5)
    assert np.all(dx == 0)


def test_softmax_flushes_non_normal_outputs_to_zero():
    # exp(-95) is a denormal float: kept by exp, flushed by the isnormal() test.
    x = np.zeros((4, 3), dtype=np.float32, order="F")
    x[1, 0] = -95.0      # denormal result -> 0
    x[2, 0] = -200.0     # underflows to 0 anyway
    x[:, 1] = [50, -45, 50, -41]   # 2 maxima: exp(-95)/2, exp(-91)/2
    x[:, 2] = np.nan     # a NaN column: every entry fails isnormal -> 0
    y = orc.softmax_fwd(x)
    assert y[1, 0] == 0.0 and y[2, 0] == 0.0 and abs(y[0, 0] - 0.5) < 1e-7
    assert y[1, 1] == 0.0 and y[3, 1] == 0.0
    assert np.all(y[:, 2] == 0.0)
    # the channelwise layer has no such flush: the denormal survives
    yc = orc.channelwise_softmax_fwd(np.asfortranarray(x[:, :1]), 1, 4, 4)
    assert 0 < yc[1, 0] < np.finfo(np.float32).tiny


def test_softmax_shift_invariance_and_log_relation():
    rng = np.random.default_rng(4)
    x = np.asfortranarray(rng.normal(0, 2, size=(40, 6)))
    y = orc.softmax_fwd(x)
    assert rel_err(orc.softmax_fwd(x + 7.25), y) < 1e-13
    assert rel_err(orc.log_softmax_fwd(x), np.log(y)) < 1e-13
    t = torch.softmax(torch.tensor(x), dim=0).numpy()
    assert rel_err(y, t) < 1e-14


# ================================================================== backward
def _fd(f, x, h=1e-5):
    """5-point central difference of scalar f at every entry of x (float64)."""
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        x0 = x[i]
        v = []
        for k in (-2, -1, 1, 2):
            x[i] = x0 + k * h
            v.append(f())
        x[i] = x0
        g[i] = (v[0] - 8 * v[1] + 8 * v[2] - v[3]) / (12 * h)
    return g


@pytest.mark.parametrize("affine", [False, True])
@pytest.mark.parametrize("G,n", [(1, 12), (3, 4)])
def test_layer_norm_bwd_finite_difference(affine, G, n):
    rng = np.random.default_rng(10 + G)
    h, w = G * n, 3
    x = np.asfortranarray(rng.normal(0.3, 1.5, size=(h, w)))
    dy = np.asfortranarray(rng.normal(size=(h, w)))
    gamma = rng.normal(1, 0.4, size=n) if affine else None
    beta = rng.normal(0, 0.4, size=n) if affine else None
    eps = 1e-3

    def loss():
        y, _ = orc.layer_norm_fwd(x, G, n, n, eps, gamma, beta)
        return float(np.sum(y * dy))

    _, stats = orc.layer_norm_fwd(x, G, n, n, eps, gamma, beta)
    dx, sgrad, dg, db = orc.layer_norm_bwd(x, dy, stats, G, n, n, eps, gamma, affine, affine)
    assert rel_err(dx, _fd(loss, x)) < 1e-7
    # every group's input gradient sums to zero (output is shift invariant)
    assert np.abs(dx.reshape(n, -1, order="F").sum(axis=0)).max() < 1e-12
    if affine:
        assert rel_err(dg, _fd(loss, gamma)) < 1e-8
        assert rel_err(db, _fd(loss, beta)) < 1e-8
    # statistics gradients: derivative of the loss with mean and variance treated as
    # free variables of y = (x-mean)/sqrt(var+eps)*gamma+beta
    mean, var = stats[:G].copy(), stats[G:].copy()
    xr = x.reshape(n, G, w, order="F")
    dyr = dy.reshape(n, G, w, order="F")
    gam = (gamma if affine else np.ones(n))[:, None, None]

    def loss_mv():
        return float(np.sum((xr - mean[None]) / np.sqrt(var[None] + eps) * gam * dyr))

    assert rel_err(sgrad[:G], _fd(loss_mv, mean)) < 1e-7
    assert rel_err(sgrad[G:], _fd(loss_mv, var, h=1e-6)) < 1e-6


def test_layer_norm_bwd_matches_torch_autograd():
    rng = np.random.default_rng(11)
    xs, dys = rng.normal(size=(5, 3, 8)), rng.normal(size=(5, 3, 8))
    g, b = rng.normal(1, 0.3, 8), rng.normal(0, 0.3, 8)
    tx = torch.tensor(xs, requires_grad=True)
    tg, tb = torch.tensor(g, requires_grad=True), torch.tensor(b, requires_grad=True)
    torch.nn.functional.layer_norm(tx, (8,), tg, tb, 1e-5).backward(torch.tensor(dys))
    x, dy = F(xs.reshape(5, -1)), F(dys.reshape(5, -1))
    _, stats = orc.layer_norm_fwd(x, 3, 8, 8, 1e-5, g, b)
    dx, _, dg, db = orc.layer_norm_bwd(x, dy, stats, 3, 8, 8, 1e-5, g, True, True)
    assert rel_err(dx.T.reshape(xs.shape), tx.grad.numpy()) < 1e-11
    assert rel_err(dg, tg.grad.numpy()) < 1e-12
    assert rel_err(db, tb.grad.numpy()) < 1e-12


@pytest.mark.parametrize("bessel", [False, True])
def test_batch_norm_bwd_finite_difference(bessel):
    rng = np.random.default_rng(12)
    C, cs, w = 3, 4, 5
    x = np.asfortranarray(rng.normal(2, 3, size=(C * cs, w)))
    dy = np.asfortranarray(rng.normal(size=(C * cs, w)))
    gamma, beta = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.1, C)
    eps = 1e-3

    def fwd():
        return orc.batch_norm_fwd(x, C, cs, eps, 0.9, gamma, beta, np.zeros(C), np.ones(C), bessel=bessel)

    def loss():
        return float(np.sum(fwd()[0] * dy))

    _, mean, var = fwd()
    dx, dg, db, dmean, dvar = orc.batch_norm_bwd(x, dy, C, cs, eps, mean, var, gamma, bessel=bessel)
    assert rel_err(dx, _fd(loss, x)) < 1e-7
    assert rel_err(dg, _fd(loss, gamma)) < 1e-8
    assert rel_err(db, _fd(loss, beta)) < 1e-8
    assert np.abs(dx.reshape(cs, C, w, order="F").sum(axis=(0, 2))).max() < 1e-12
    m, v = mean.copy(), var.copy()
    xr, dyr = x.reshape(cs, C, w, order="F"), dy.reshape(cs, C, w, order="F")

    def loss_mv():
        return float(np.sum(((xr - m[None, :, None]) / np.sqrt(v[None, :, None] + eps) * gamma[None, :, None]) * dyr))

    assert rel_err(dmean, _fd(loss_mv, m)) < 1e-7
    assert rel_err(dvar, _fd(loss_mv, v, h=1e-6)) < 1e-6
    # inference mode: statistics are constants; their gradients are reported as zero
    rm, rv = rng.normal(size=C), rng.uniform(0.5, 2, C)
    dxi, dgi, dbi, dmi, dvi = orc.batch_norm_bwd(x, dy, C, cs, eps, mean, var, gamma, rm, rv,
                                                 bessel=bessel, training=False)
    assert np.all(dmi == 0) and np.all(dvi == 0)
    assert rel_err(dbi, dyr.sum(axis=(0, 2))) < 1e-13


def test_batch_norm_bwd_matches_torch_autograd():
    rng = np.random.default_rng(13)
    N, C, H, W = 4, 3, 2, 5
    xs, dys = rng.normal(2, 3, size=(N, C, H, W)), rng.normal(size=(N, C, H, W))
    g, b = rng.uniform(0.5, 1.5, C), rng.normal(0, 0.1, C)
    tx = torch.tensor(xs, requires_grad=True)
    tg, tb = torch.tensor(g, requires_grad=True), torch.tensor(b, requires_grad=True)
    torch.nn.functional.batch_norm(tx, None, None, tg, tb, training=True, eps=1e-5).backward(torch.tensor(dys))
    x, dy = F(xs.reshape(N, -1)), F(dys.reshape(N, -1))
    _, mean, var = orc.batch_norm_fwd(x, C, H * W, 1e-5, 0.9, g, b, np.zeros(C), np.ones(C), bessel=False)
    dx, dg, db, _, _ = orc.batch_norm_bwd(x, dy, C, H * W, 1e-5, mean, var, g, bessel=False)
    assert rel_err(dx.T.reshape(xs.shape), tx.grad.numpy()) < 1e-11
    assert rel_err(dg, tg.grad.numpy()) < 1e-12
    assert rel_err(db, tb.grad.numpy()) < 1e-12


@pytest.mark.parametrize("kind", ["softmax", "log_softmax", "channelwise"])
def test_softmax_family_bwd(kind):
    rng = np.random.default_rng(14)
    h, w = 12, 4
    x = np.asfortranarray(rng.normal(0, 2, size=(h, w)))
    dy = np.asfortranarray(rng.normal(size=(h, w)))
    tx = torch.tensor(x, requires_grad=True)
    if kind == "softmax":
        y = orc.softmax_fwd(x)
        dx = orc.softmax_bwd(y, dy)
        torch.softmax(tx, dim=0).backward(torch.tensor(dy))
        loss = lambda: float(np.sum(orc.softmax_fwd(x) * dy))
    elif kind == "log_softmax":
        y = orc.log_softmax_fwd(x)
        dx = orc.log_softmax_bwd(y, dy)
        torch.log_softmax(tx, dim=0).backward(torch.tensor(dy))
        loss = lambda: float(np.sum(orc.log_softmax_fwd(x) * dy))
    else:
        y = orc.channelwise_softmax_fwd(x, 3, 4, 4)
        dx = orc.channelwise_softmax_bwd(y, dy, 3, 4, 4)
        torch.softmax(tx.reshape(3, 4, w), dim=1).reshape(h, w).backward(torch.tensor(dy))
        loss = lambda: float(np.sum(orc.channelwise_softmax_fwd(x, 3, 4, 4) * dy))
    assert rel_err(dx, tx.grad.numpy()) < 1e-12
    assert rel_err(dx, _fd(loss, x)) < 1e-7
    if kind == "softmax":
        assert np.abs(dx.sum(axis=0)).max() < 1e-13
    if kind == "channelwise":
        assert np.abs(dx.reshape(4, -1, order="F").sum(axis=0)).max() < 1e-13


def test_leading_dimension_and_f32_f64_agreement():
    """Views with ld > height must give the same numbers as packed matrices."""
    rng = np.random.default_rng(15)
    big = np.asfortranarray(rng.normal(size=(40, 6)).astype(np.float32))
    view = big[4:28, :]
    packed = np.asfortranarray(view.copy())
    assert view.strides[1] // 4 == 40
    assert np.array_equal(orc.softmax_fwd(view), orc.softmax_fwd(packed))
    assert np.array_equal(orc.log_softmax_fwd(view), orc.log_softmax_fwd(packed))
    assert np.array_equal(orc.layer_norm_fwd(view, 2, 12, 12, 1e-5)[0], orc.layer_norm_fwd(packed, 2, 12, 12, 1e-5)[0])
    assert np.array_equal(orc.channelwise_softmax_fwd(view, 4, 6, 6), orc.channelwise_softmax_fwd(packed, 4, 6, 6))
    g, b = np.ones(3, np.float32), np.zeros(3, np.float32)
    a = orc.batch_norm_fwd(view, 3, 8, 1e-5, 0.9, g, b, np.zeros(3, np.float32), np.ones(3, np.float32))[0]
    c = orc.batch_norm_fwd(packed, 3, 8, 1e-5, 0.9, g, b, np.zeros(3, np.float32), np.ones(3, np.float32))[0]
    assert np.array_equal(a, c)
    y64 = orc.softmax_fwd(packed.astype(np.float64, order="F"))
    assert rel_err(orc.softmax_fwd(packed), y64) < 1e-6


# ============================================================== instance norm
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-12)])
def test_instance_norm_golden(golden, dt, tol):
    x = F(golden["in_x"], dt)
    y, sums = orc.instance_norm_fwd(x, 5, 21, 1e-5)
    assert rel_err(y.T, golden["in_y"]) < tol
    val = float(golden["in_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS   # the reference test's acceptance band
    xd = golden["in_x"].astype(np.float64).reshape(15, 5, 21)
    assert rel_err(sums[:5].T, xd.sum(axis=2)) < 10 * tol
    assert rel_err(sums[5:].T, (xd * xd).sum(axis=2)) < 10 * tol


def test_instance_norm_matches_torch_and_layer_norm():
    rng = np.random.default_rng(21)
    C, cs, w = 4, 9, 6
    x = np.asfortranarray(rng.normal(0.5, 2.0, size=(C * cs, w)))
    dy = np.asfortranarray(rng.normal(size=(C * cs, w)))
    y, sums = orc.instance_norm_fwd(x, C, cs, 1e-5)
    dx = orc.instance_norm_bwd(x, dy, sums, C, cs, 1e-5)
    xt = torch.tensor(x.T.reshape(w, C, cs), requires_grad=True)
    yt = torch.nn.functional.instance_norm(xt, eps=1e-5)
    yt.backward(torch.tensor(dy.T.reshape(w, C, cs)))
    assert rel_err(y.T.reshape(w, C, cs), yt.detach().numpy()) < 1e-13
    assert rel_err(dx.T.reshape(w, C, cs), xt.grad.numpy()) < 1e-12
    # the same numbers as layer norm over groups of cs entries, without scale and bias
    y2, stats = orc.layer_norm_fwd(x, C, cs, cs, 1e-5)
    dx2, _, _, _ = orc.layer_norm_bwd(x, dy, stats, C, cs, cs, 1e-5)
    assert rel_err(y, y2) < 1e-13 and rel_err(dx, dx2) < 1e-12


def test_instance_norm_bwd_finite_difference_and_single_entry_channels():
    rng = np.random.default_rng(22)
    C, cs, w = 3, 5, 2
    x = np.asfortranarray(rng.normal(0.3, 1.5, size=(C * cs, w)))
    dy = np.asfortranarray(rng.normal(size=(C * cs, w)))
    eps = 1e-3

    def loss():
        return float(np.sum(orc.instance_norm_fwd(x, C, cs, eps)[0] * dy))

    _, sums = orc.instance_norm_fwd(x, C, cs, eps)
    dx = orc.instance_norm_bwd(x, dy, sums, C, cs, eps)
    assert rel_err(dx, _fd(loss, x)) < 1e-7
    assert np.abs(dx.reshape(cs, -1, order="F").sum(axis=0)).max() < 1e-12
    # channels of one entry: constant output, zero gradient (instance_norm.cpp:65-68, :164-167)
    x1 = np.asfortranarray(rng.normal(size=(7, 3)).astype(np.float32))
    y1, s1 = orc.instance_norm_fwd(x1, 7, 1, 1e-5)
    assert not y1.any() and not orc.instance_norm_bwd(x1, x1, s1, 7, 1, 1e-5).any()


# ====================================================== entry-wise batch norm
@pytest.mark.parametrize("tag,rows", [("mb14", 14), ("all29", 29)])
def test_entrywise_batch_norm_golden(golden, tag, rows):
    for dt, tol in ((np.float32, 3e-6), (np.float64, 1e-12)):
        x = F(golden["ebn_x"][:rows], dt)
        rm, rv = np.zeros(105, dt), np.ones(105, dt)
        y, stats = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, rm, rv)
        assert rel_err(y.T, golden[f"ebn_{tag}_y"]) < tol
        assert rel_err(stats[:, 0], golden[f"ebn_{tag}_mean"]) < tol
        assert rel_err(stats[:, 1], golden[f"ebn_{tag}_var"]) < 10 * tol
        # running statistics: exponential moving average from (0, 1) with decay 0.9
        assert rel_err(rm, 0.1 * golden[f"ebn_{tag}_mean"]) < 10 * tol
        assert rel_err(rv, 0.9 + 0.1 * golden[f"ebn_{tag}_var"]) < 10 * tol


def test_entrywise_batch_norm_matches_torch_autograd_and_inference():
    rng = np.random.default_rng(31)
    h, w = 23, 11
    x = np.asfortranarray(rng.normal(0.5, 2.0, size=(h, w)))
    dy = np.asfortranarray(rng.normal(size=(h, w)))
    rm, rv = rng.normal(size=h), rng.uniform(0.5, 2.0, size=h)
    rm0, rv0 = rm.copy(), rv.copy()
    y, stats = orc.entrywise_batch_norm_fwd(x, 0.8, 1e-4, rm, rv)
    xt = torch.tensor(x.T, requires_grad=True)
    yt = (xt - xt.mean(0)) / torch.sqrt(xt.var(0, unbiased=True) + 1e-4)
    yt.backward(torch.tensor(dy.T))
    dx, _ = orc.entrywise_batch_norm_bwd(x, dy, stats, 1e-4)
    assert rel_err(y.T, yt.detach().numpy()) < 1e-13 and rel_err(dx.T, xt.grad.numpy()) < 1e-12
    assert rel_err(rm, 0.8 * rm0 + 0.2 * x.mean(1)) < 1e-13
    assert rel_err(rv, 0.8 * rv0 + 0.2 * x.var(1, ddof=1)) < 1e-13
    # inference: running statistics in, nothing updated, gradient is dy / stdev
    rm1, rv1 = rm.copy(), rv.copy()
    yi, _ = orc.entrywise_batch_norm_fwd(x, 0.8, 1e-4, rm1, rv1, training=False)
    assert rel_err(yi, (x - rm[:, None]) / np.sqrt(rv[:, None] + 1e-4)) < 1e-13
    assert np.array_equal(rm1, rm) and np.array_equal(rv1, rv)
    dxi, _ = orc.entrywise_batch_norm_bwd(x, dy, stats, 1e-4, rv, training=False)
    assert rel_err(dxi, dy / np.sqrt(rv[:, None] + 1e-4)) < 1e-13


def test_entrywise_batch_norm_reference_variance_is_not_clamped():
    """E[x^2] - mean^2 in fp32 can come out negative for a pair of nearly equal large values;
    the reference keeps that value (entrywise_batch_normalization.cpp:118, no clamp), times the
    Bessel factor, and its output for that entry is then NaN once var + epsilon < 0.  The GPU
    kernels clamp the difference at zero instead (a documented deviation, checked by
    tests/test_gpu_parity.py::test_entrywise_batch_norm_clamps_negative_variance)."""
    x = np.asfortranarray(np.array([[3198.374755859375, 3198.375], [1.0, 3.0]], dtype=np.float32))
    rm, rv = np.zeros(2, np.float32), np.ones(2, np.float32)
    y, stats = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, rm, rv)
    assert stats[0, 1] == np.float32(-2.0)            # (-1) * w / (w - 1) with w = 2
    assert np.isnan(y[0]).all()                       # 1 / sqrt(-2 + 1e-5)
    assert stats[1, 1] == np.float32(2.0) and np.isfinite(y[1]).all()   # the ordinary row is untouched
    assert rv[0] == np.float32(0.9) * np.float32(1.0) + (np.float32(1.0) - np.float32(0.9)) * np.float32(-2.0)


def test_entrywise_batch_norm_bwd_finite_difference_and_single_sample():
    rng = np.random.default_rng(32)
    h, w = 4, 5
    x = np.asfortranarray(rng.normal(0.3, 1.5, size=(h, w)))
    dy = np.asfortranarray(rng.normal(size=(h, w)))
    eps = 1e-3

    def loss():
        return float(np.sum(orc.entrywise_batch_norm_fwd(x, 0.9, eps, np.zeros(h), np.ones(h))[0] * dy))

    _, stats = orc.entrywise_batch_norm_fwd(x, 0.9, eps, np.zeros(h), np.ones(h))
    dx, sgrad = orc.entrywise_batch_norm_bwd(x, dy, stats, eps)
    assert rel_err(dx, _fd(loss, x)) < 1e-7
    assert np.abs(dx.sum(axis=1)).max() < 1e-12          # every entry's gradient sums to zero over the batch
    mean, var = stats[:, 0].copy(), stats[:, 1].copy()

    def loss_mv():
        return float(np.sum((x - mean[:, None]) / np.sqrt(var[:, None] + eps) * dy))

    assert rel_err(sgrad[:, 0], _fd(loss_mv, mean)) < 1e-7
    assert rel_err(sgrad[:, 1], _fd(loss_mv, var, h=1e-6)) < 1e-6
    # one sample: variance 1, running statistics untouched, zero gradient
    # (entrywise_batch_normalization.cpp:103-106, :257-261)
    x1 = np.asfortranarray(rng.normal(size=(6, 1)).astype(np.float32))
    rm, rv = np.full(6, 0.25, np.float32), np.full(6, 2.0, np.float32)
    y1, s1 = orc.entrywise_batch_norm_fwd(x1, 0.9, 1e-5, rm, rv)
    assert not y1.any() and np.array_equal(s1[:, 0], x1[:, 0]) and (s1[:, 1] == 1).all()
    assert (rm == 0.25).all() and (rv == 2.0).all()
    assert not orc.entrywise_batch_norm_bwd(x1, x1, s1, 1e-5)[0].any()


# ============================================================== cross entropy
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-12)])
def test_cross_entropy_golden(golden, dt, tol):
    x = F(golden["ce_prediction"], dt)
    dense, labels = F(golden["ce_dense_truth"], dt), F(golden["ce_labels"], dt)
    loss = orc.cross_entropy_fwd(x, dense)
    assert rel_err(loss, golden["ce_loss_dense"]) < tol
    val = float(golden["ce_metric_dense"])
    assert abs(np.mean((1e-3 * loss.astype(np.float64)) ** 2) - val) <= val * float(golden["ce_metric_tol"])
    loss = orc.cross_entropy_fwd(x, labels, use_labels=True)
    assert rel_err(loss, golden["ce_loss_labels"]) < tol
    val = float(golden["ce_metric_labels"])
    assert abs(np.mean((1e-3 * loss.astype(np.float64)) ** 2) - val) <= val * float(golden["ce_metric_tol"])


def test_cross_entropy_backward_matches_autograd_and_skips_nonpositive_truth():
    rng = np.random.default_rng(5)
    h, w = 24, 7
    x = np.asfortranarray(rng.uniform(0.25, 1.0, (h, w)))
    truth = np.asfortranarray(rng.uniform(-0.5, 1.0, (h, w)))   # a third of the entries <= 0
    truth[3, 2] = 0.0
    dy = rng.standard_normal(w)
    loss = orc.cross_entropy_fwd(x, truth)
    pos = truth > 0
    assert np.allclose(loss, -(np.where(pos, truth, 0.0) * np.log(x)).sum(axis=0), rtol=1e-13)
    dx, dtruth = orc.cross_entropy_bwd(x, truth, dy)
    tx = torch.tensor(x, requires_grad=True)
    tt = torch.tensor(truth, requires_grad=True)
    obj = (-(tt * torch.log(tx)) * torch.tensor(dy)).sum()
    gx, gt = torch.autograd.grad(obj, (tx, tt))
    assert np.allclose(dx[pos], gx.numpy()[pos], rtol=1e-12)
    assert np.all(dx[~pos] == 0.0)                       # the reference zeroes them (xhat > 0 test)
    assert np.allclose(dtruth, gt.numpy(), rtol=1e-12)   # dxhat = -dy log x everywhere
    # labels: one class index per spatial position, prediction rows are class-major
    classes, spatial = 4, 6
    x = np.asfortranarray(rng.uniform(0.25, 1.0, (classes * spatial, w)))
    lab = rng.integers(0, classes, (spatial, w))
    onehot = np.zeros((classes, spatial, w))
    for c in range(w):
        onehot[lab[:, c], np.arange(spatial), c] = 1.0
    onehot = np.asfortranarray(onehot.reshape(classes * spatial, w))
    labf = np.asfortranarray(lab.astype(np.float64))
    assert np.array_equal(orc.cross_entropy_fwd(x, labf, use_labels=True), orc.cross_entropy_fwd(x, onehot))
    dxl, none = orc.cross_entropy_bwd(x, labf, dy, use_labels=True)
    assert none is None
    assert np.array_equal(dxl, orc.cross_entropy_bwd(x, onehot, dy)[0])


# ============================================================ scale/bias layers
@pytest.mark.parametrize("dt,tol", [(np.float32, 2e-6), (np.float64, 1e-12)])
def test_scale_bias_golden(golden, dt, tol):
    x = F(golden["esb_x"], dt)
    wts = np.asfortranarray(np.stack([golden["esb_scale"], golden["esb_bias"]], axis=1).astype(dt))
    y = orc.entrywise_scale_bias_fwd(x, wts)
    assert rel_err(y.T, golden["esb_y"]) < tol
    val = float(golden["esb_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS
    x = F(golden["csb_x"], dt)
    wts = np.asfortranarray(np.stack([golden["csb_scale"], golden["csb_bias"]], axis=1).astype(dt))
    y = orc.channelwise_scale_bias_fwd(x, wts, 7, 15)
    assert rel_err(y.T, golden["csb_y"]) < tol
    val = float(golden["csb_metric"])
    assert abs(metric(y) - val) <= 8 * val * F32_EPS


def test_scale_bias_backward_matches_autograd():
    rng = np.random.default_rng(11)
    C, cs, w = 5, 6, 9
    h = C * cs
    x = np.asfortranarray(rng.standard_normal((h, w)))
    dy = np.asfortranarray(rng.standard_normal((h, w)))
    tx = torch.tensor(x, requires_grad=True)
    tdy = torch.tensor(dy)
    # entry-wise: one (scale, bias) per row
    wts = np.asfortranarray(rng.standard_normal((h, 2)))
    tw = torch.tensor(wts, requires_grad=True)
    y = tw[:, 0:1] * tx + tw[:, 1:2]
    assert np.allclose(orc.entrywise_scale_bias_fwd(x, wts), y.detach().numpy(), rtol=1e-13)
    gx, gw = torch.autograd.grad((y * tdy).sum(), (tx, tw))
    dx, wg = orc.entrywise_scale_bias_bwd(x, dy, wts)
    assert np.allclose(dx, gx.numpy(), rtol=1e-12) and np.allclose(wg, gw.numpy(), rtol=1e-11, atol=1e-13)
    # channel-wise: one (scale, bias) per block of cs rows
    wts = np.asfortranarray(rng.standard_normal((C, 2)))
    tw = torch.tensor(wts, requires_grad=True)
    y = tw[:, 0].repeat_interleave(cs)[:, None] * tx + tw[:, 1].repeat_interleave(cs)[:, None]
    assert np.allclose(orc.channelwise_scale_bias_fwd(x, wts, C, cs), y.detach().numpy(), rtol=1e-13)
    gx, gw = torch.autograd.grad((y * tdy).sum(), (tx, tw))
    dx, wg = orc.channelwise_scale_bias_bwd(x, dy, wts, C, cs)
    assert np.allclose(dx, gx.numpy(), rtol=1e-12) and np.allclose(wg, gw.numpy(), rtol=1e-11, atol=1e-13)


# ------------------------------------------------------------- gradient buffer update
def test_gradient_sink_against_elementwise_arithmetic():
    """Scale + Axpy of optimizer::add_to_gradient, checked against numpy's own float32
    arithmetic (each product and the sum rounded once) and against what the two library
    calls fix: a scale of zero discards NaN/Inf already in the buffer, a scale of one
    leaves the buffer's bits alone, a product of -0 lands as +0 on a zeroed buffer."""
    rng = np.random.default_rng(207)
    h, w = 37, 5
    g = np.asfortranarray(rng.standard_normal((h, w)).astype(np.float32))
    c = np.asfortranarray(rng.standard_normal((h, w)).astype(np.float32))
    a = np.float32(0.37)
    # ready buffer: g + a * c
    out = orc.gradient_sink(g, c, 1.0, a)
    assert out.tobytes() == (g + a * c).astype(np.float32).tobytes()
    # general factor: two roundings on the buffer side
    b = np.float32(-1.25)
    out = orc.gradient_sink(g, c, b, a)
    assert out.tobytes() == ((b * g).astype(np.float32) + (a * c).astype(np.float32)).tobytes()
    # cleared buffer: contents are not read
    dirty = g.copy(order="F")
    dirty[3, 1], dirty[0, 0], dirty[5, 4] = np.nan, np.inf, -np.inf
    out = orc.gradient_sink(dirty, c, 0.0, a)
    assert out.tobytes() == (np.float32(0) + (a * c).astype(np.float32)).tobytes()
    assert np.isfinite(out).all()
    zc = np.zeros((h, w), dtype=np.float32, order="F")
    zc[2, 2] = -0.0
    out = orc.gradient_sink(dirty, zc, 0.0, 1.0)
    assert not np.signbit(out).any()
    # the input gradient is not modified, the contribution's padding is skipped
    wide = np.asfortranarray(rng.standard_normal((h + 3, w)).astype(np.float32))
    out = orc.gradient_sink(g, wide[:h], 1.0, 2.0)
    assert np.array_equal(out, g + np.float32(2) * wide[:h])
    # float64 instance
    out = orc.gradient_sink(g.astype(np.float64), c.astype(np.float64), 1.0, 0.5)
    assert np.array_equal(out, g.astype(np.float64) + 0.5 * c.astype(np.float64))


def test_gradient_buffer_status_machine():
    """get_gradient_buffer's choice of factors (optimizer_impl.hpp:219-288) on the host."""
    from lbann_amd.layers import gradient_buffer as GB
    b = GB.__new__(GB)
    b.status = GB.CLEARED
    assert b._scales(False) == (0.0, 1.0) and b.status == GB.READY
    assert b._scales(False) == (1.0, 1.0) and b.status == GB.READY
    assert b._scales(True) == (1.0, 1.0) and b.status == GB.SYNC_NEEDED
    assert b._scales(False) == (1.0, 1.0) and b.status == GB.SYNC_NEEDED
    b.finish_sync()
    assert b.status == GB.READY
    b.clear()
    assert b._scales(True) == (0.0, 1.0) and b.status == GB.SYNC_NEEDED
    b.status = "bogus"
    with pytest.raises(ValueError):
        b._scales(False)
