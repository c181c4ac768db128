"""Seeded sweep over small random shapes, leading dimensions and layer options: every
layer, GPU through the C ABI against the CPU oracle.  The shapes are drawn so that the
vector kernels, their masked variants and the scalar fallbacks are all hit (lengths that
are and are not multiples of 4 or 8, padded leading dimensions, single rows and columns)."""
import os

import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import TOL_F16, TOL_F32, check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()
    assert torch.cuda.is_available()
    return layers


def f64(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float64))


def f32(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float32))


def rand(rng, h, w, mean=0.0, std=1.0):
    return np.asfortranarray((rng.standard_normal((w, h)) * std + mean).astype(np.float32).T)


def draw_length(rng):
    """Mostly vector-friendly lengths, some odd ones, a few long ones."""
    kind = rng.integers(0, 10)
    if kind < 5:
        return int(rng.integers(1, 400)) * 8
    if kind < 8:
        return int(rng.integers(1, 3000))
    return int(rng.integers(3000, 40000))


# LBN_RANDOM_CASES widens the sweep for a one-off soak; the default keeps the suite short
CASES = list(range(int(os.environ.get("LBN_RANDOM_CASES", "24"))))


@pytest.mark.parametrize("case", CASES)
def test_softmax_family_random(L, case):
    rng = np.random.default_rng(1000 + case)
    n, w = draw_length(rng), int(rng.integers(1, 40))
    pad = int(rng.choice([0, 0, 4, 3]))
    x, dy = rand(rng, n, w, 0.0, 2.5), rand(rng, n, w)
    for kind, layer, fwd, bwd in (("softmax", L.softmax_layer(), orc.softmax_fwd, orc.softmax_bwd),
                                  ("log_softmax", L.log_softmax_layer(), orc.log_softmax_fwd, orc.log_softmax_bwd)):
        y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=n + pad)).to_numpy()
        dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=n + pad)).to_numpy()
        check(f"{kind} y n={n} w={w} pad={pad}", y, fwd(x), fwd(f64(x)))
        check(f"{kind} dx n={n} w={w} pad={pad}", dx, bwd(y, dy), bwd(f64(y), f64(dy)))


@pytest.mark.parametrize("case", CASES)
def test_softmax_f16_and_fused_cross_entropy_random(L, case):
    """fp16-storage softmax / log-softmax (2e-3 against the fp32 oracle on the rounded values) and
    the fused softmax + cross-entropy forward (oracle: the composition of the two restatements),
    dense ground truth and class labels, on the same random shapes."""
    rng = np.random.default_rng(7000 + case)
    n, w = draw_length(rng), int(rng.integers(1, 40))
    pad = int(rng.choice([0, 0, 8, 3]))
    x, dy = rand(rng, n, w, 0.0, 2.5), rand(rng, n, w)
    xh = f32(x.astype(np.float16))
    dyh = f32(dy.astype(np.float16))
    for kind, layer, fwd, bwd in (("softmax", L.softmax_layer(), orc.softmax_fwd, orc.softmax_bwd),
                                  ("log_softmax", L.log_softmax_layer(), orc.log_softmax_fwd, orc.log_softmax_bwd)):
        y = layer.forward(L.DeviceMatrix.from_numpy(xh, dtype=torch.float16, ldim=n + pad)).to_numpy()
        check(f"random f16 {kind} y {n}x{w}", y, fwd(xh), fwd(f64(xh)), tol=TOL_F16)
        dx = layer.backward(L.DeviceMatrix.from_numpy(dyh, dtype=torch.float16, ldim=n + pad)).to_numpy()
        yh = f32(y)
        check(f"random f16 {kind} dx {n}x{w}", dx, bwd(yh, dyh), bwd(f64(yh), f64(dyh)), tol=TOL_F16)
    # fused forward: dense ground truth
    truth = np.asfortranarray(rng.random((n, w)).astype(np.float32))
    truth[rng.random((n, w)) < 0.5] = 0.0
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((n,))
    y, loss = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x, ldim=n + pad),
                                              L.DeviceMatrix.from_numpy(truth, ldim=n + pad))
    y_ref, y64 = orc.softmax_fwd(x), orc.softmax_fwd(f64(x))
    check(f"random fused y {n}x{w}", y.to_numpy(), y_ref, y64)
    check(f"random fused loss {n}x{w}", loss.to_numpy()[0], orc.cross_entropy_fwd(y_ref, truth),
          orc.cross_entropy_fwd(y64, f64(truth)))
    # fused backward: the composition of the two restated backward passes on the y the GPU wrote
    g = rng.standard_normal(w).astype(np.float32)
    yg = y.to_numpy()
    dx = L.softmax_cross_entropy_backward(sm, ce, L.DeviceMatrix.from_numpy(g.reshape(1, w)), want_dtruth=bool(case % 2))
    dp_ref, dt_ref = orc.cross_entropy_bwd(yg, truth, g)
    dp64, dt64 = orc.cross_entropy_bwd(f64(yg), f64(truth), g.astype(np.float64))
    check(f"random fused dx {n}x{w}", dx.to_numpy(), orc.softmax_bwd(yg, dp_ref), orc.softmax_bwd(f64(yg), dp64))
    if case % 2:
        check(f"random fused dtruth {n}x{w}", ce.error_signals[1].to_numpy(), dt_ref, dt64)
    # class labels, one per column
    labels = np.asfortranarray(rng.integers(0, n, (1, w)).astype(np.float32))
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((n, 1), use_labels=True)
    y, loss = L.softmax_cross_entropy_forward(sm, ce, L.DeviceMatrix.from_numpy(x, ldim=n + pad),
                                              L.DeviceMatrix.from_numpy(labels))
    check(f"random fused labels loss {n}x{w}", loss.to_numpy()[0], orc.cross_entropy_fwd(y_ref, labels, True),
          orc.cross_entropy_fwd(y64, f64(labels), True))
    yg = y.to_numpy()
    dx = L.softmax_cross_entropy_backward(sm, ce, L.DeviceMatrix.from_numpy(g.reshape(1, w)))
    dp_ref, _ = orc.cross_entropy_bwd(yg, labels, g, True)
    dp64, _ = orc.cross_entropy_bwd(f64(yg), f64(labels), g.astype(np.float64), True)
    check(f"random fused labels dx {n}x{w}", dx.to_numpy(), orc.softmax_bwd(yg, dp_ref), orc.softmax_bwd(f64(yg), dp64))


@pytest.mark.parametrize("case", CASES)
def test_channelwise_softmax_and_instance_norm_random(L, case):
    rng = np.random.default_rng(2000 + case)
    C, cs, w = int(rng.integers(1, 12)), min(draw_length(rng), 6000), int(rng.integers(1, 12))
    h = C * cs
    pad = int(rng.choice([0, 0, 4, 1]))
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    cw = L.channelwise_softmax_layer((C, cs))
    y = cw.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = cw.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    check(f"channelwise y C={C} cs={cs} w={w}", y, orc.channelwise_softmax_fwd(x, C, cs, cs),
          orc.channelwise_softmax_fwd(f64(x), C, cs, cs))
    check(f"channelwise dx C={C} cs={cs} w={w}", dx, orc.channelwise_softmax_bwd(y, dy, C, cs, cs),
          orc.channelwise_softmax_bwd(f64(y), f64(dy), C, cs, cs))
    inl = L.instance_norm_layer((C, cs), 1e-5)
    y = inl.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = inl.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    y32, s32 = orc.instance_norm_fwd(x, C, cs, 1e-5)
    y64, s64 = orc.instance_norm_fwd(f64(x), C, cs, 1e-5)
    check(f"instance norm y C={C} cs={cs} w={w}", y, y32, y64)
    check(f"instance norm dx C={C} cs={cs} w={w}", dx, orc.instance_norm_bwd(x, dy, s32, C, cs, 1e-5),
          orc.instance_norm_bwd(f64(x), f64(dy), s64, C, cs, 1e-5))


@pytest.mark.parametrize("case", CASES)
def test_layer_norm_random(L, case):
    rng = np.random.default_rng(3000 + case)
    G, n, w = int(rng.choice([1, 1, 2, 5])), min(draw_length(rng), 20000), int(rng.integers(1, 30))
    half = bool(case % 3 == 2)
    affine = bool(case % 2)
    h = G * n
    pad = int(rng.choice([0, 0, 8, 2]))
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    if half:
        x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
    g = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32) if affine else None
    b = (0.2 * rng.standard_normal(n)).astype(np.float32) if affine else None
    kw = dict(scale_values=g, bias_values=b) if affine else {}
    dims, sd = ((G, n), 1) if G > 1 else ((n,), 0)
    layer = L.layer_norm_layer(dims, 1e-5, affine, affine, sd, **kw)
    tdt = torch.float16 if half else torch.float32
    tol = TOL_F16 if half else TOL_F32
    y = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=h + pad)).to_numpy()
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        gg = None if g is None else conv(g)
        bb = None if b is None else conv(b)
        dst["y"], st = orc.layer_norm_fwd(conv(x), G, n, n, 1e-5, gg, bb)
        dst["dx"], _, dst["dscale"], dst["dbias"] = orc.layer_norm_bwd(conv(x), conv(dy), st, G, n, n, 1e-5, gg,
                                                                         affine, affine)
    tag = f"G={G} n={n} w={w} half={half} affine={affine} pad={pad}"
    check("layer norm y " + tag, y, ref["y"], ex["y"], tol=tol)
    if n > 1:
        check("layer norm dx " + tag, dx, ref["dx"], ex["dx"], tol=tol)
    if affine:
        check("layer norm dscale " + tag, layer.m_scale_gradient.to_numpy(), ref["dscale"], ex["dscale"], tol=tol)
        check("layer norm dbias " + tag, layer.m_bias_gradient.to_numpy(), ref["dbias"], ex["dbias"], tol=tol)


@pytest.mark.parametrize("case", CASES)
def test_batch_norms_random(L, case):
    rng = np.random.default_rng(4000 + case)
    C, cs, w = int(rng.integers(1, 20)), min(draw_length(rng), 5000), int(rng.integers(2, 24))
    h = C * cs
    pad = int(rng.choice([0, 0, 4, 1]))
    bessel = bool(case % 2)
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (0.1 * rng.standard_normal(C)).astype(np.float32)
    bn = L.batch_normalization_layer((C, cs), 0.9, 1e-5, bessel, g, b)
    y = bn.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = bn.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        rm, rv = conv(np.zeros(C)), conv(np.ones(C))
        dst["y"], m, v = orc.batch_norm_fwd(conv(x), C, cs, 1e-5, 0.9, conv(g), conv(b), rm, rv, bessel)
        dst["dx"], dst["dscale"], dst["dbias"], _, _ = orc.batch_norm_bwd(conv(x), conv(dy), C, cs, 1e-5, m, v,
                                                                         conv(g), bessel=bessel)
    tag = f"C={C} cs={cs} w={w} bessel={bessel} pad={pad}"
    check("batch norm y " + tag, y, ref["y"], ex["y"])
    check("batch norm dx " + tag, dx, ref["dx"], ex["dx"])
    check("batch norm dscale " + tag, bn.m_scale_gradient.to_numpy(), ref["dscale"], ex["dscale"])
    check("batch norm dbias " + tag, bn.m_bias_gradient.to_numpy(), ref["dbias"], ex["dbias"])
    # entry-wise batch norm on the same data
    eb = L.entrywise_batch_normalization_layer((h,), 0.9, 1e-5)
    y = eb.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = eb.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    y32, st32 = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, np.zeros(h, np.float32), np.ones(h, np.float32))
    y64, st64 = orc.entrywise_batch_norm_fwd(f64(x), 0.9, 1e-5, np.zeros(h), np.ones(h))
    check("entrywise bn y " + tag, y, y32, y64)
    check("entrywise bn dx " + tag, dx, orc.entrywise_batch_norm_bwd(x, dy, st32, 1e-5)[0],
          orc.entrywise_batch_norm_bwd(f64(x), f64(dy), st64, 1e-5)[0])


@pytest.mark.parametrize("case", CASES)
def test_cross_entropy_and_scale_bias_random(L, case):
    rng = np.random.default_rng(5000 + case)
    C = int(rng.integers(1, 12))
    cs = draw_length(rng) // int(rng.choice([1, 4, 16])) + 1 if case % 3 else int(rng.integers(1, 60)) * 4
    h, w = C * cs, int(rng.integers(1, 70))
    pad = int(rng.choice([0, 0, 4, 3]))
    tag = f"C={C} cs={cs} w={w} pad={pad}"
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    # scale/bias layers
    for kind, n in (("entrywise", h), ("channelwise", C)):
        wts = np.asfortranarray(np.stack([rng.normal(1, 1, n), rng.normal(0, 1, n)], axis=1).astype(np.float32))
        if kind == "entrywise":
            layer = L.entrywise_scale_bias_layer((h,))
            fwd = lambda a, b: orc.entrywise_scale_bias_fwd(a, b)
            bwd = lambda a, g, b: orc.entrywise_scale_bias_bwd(a, g, b)
        else:
            layer = L.channelwise_scale_bias_layer((C, cs))
            fwd = lambda a, b: orc.channelwise_scale_bias_fwd(a, b, C, cs)
            bwd = lambda a, g, b: orc.channelwise_scale_bias_bwd(a, g, b, C, cs)
        layer.set_weights(wts[:, 0], wts[:, 1])
        y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
        dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
        check(f"{kind} scale/bias y {tag}", y, fwd(x, wts), fwd(f64(x), f64(wts)))
        rdx, rwg = bwd(x, dy, wts)
        edx, ewg = bwd(f64(x), f64(dy), f64(wts))
        check(f"{kind} scale/bias dx {tag}", dx, rdx, edx)
        check(f"{kind} scale/bias dweights {tag}", layer.m_weights_gradient.to_numpy(), rwg, ewg)
    # cross entropy, dense ground truth and labels (C classes, cs spatial positions)
    pred = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float32).T)
    dense = np.asfortranarray(rng.uniform(-0.3, 1.0, (w, h)).astype(np.float32).T)
    labels = np.asfortranarray(rng.integers(0, C, (w, cs)).astype(np.float32).T)
    dloss = rng.standard_normal(w).astype(np.float32)
    drow = L.DeviceMatrix.from_numpy(dloss.reshape(1, -1))
    for use_labels, truth, dims in ((False, dense, (h,)), (True, labels, (C, cs))):
        layer = L.cross_entropy_layer(dims, use_labels=use_labels)
        tpad = pad if truth.shape[0] + pad >= truth.shape[0] else 0
        loss = layer.forward(L.DeviceMatrix.from_numpy(pred, ldim=h + pad),
                             L.DeviceMatrix.from_numpy(truth, ldim=truth.shape[0] + tpad)).to_numpy()[0]
        check(f"cross entropy loss labels={use_labels} {tag}", loss, orc.cross_entropy_fwd(pred, truth, use_labels),
              orc.cross_entropy_fwd(f64(pred), f64(truth), use_labels))
        dx, dt = layer.backward(drow)
        rdx, rdt = orc.cross_entropy_bwd(pred, truth, dloss, use_labels)
        edx, edt = orc.cross_entropy_bwd(f64(pred), f64(truth), dloss.astype(np.float64), use_labels)
        check(f"cross entropy dx labels={use_labels} {tag}", dx.to_numpy(), rdx, edx)
        if not use_labels:
            check(f"cross entropy dtruth {tag}", dt.to_numpy(), rdt, edt)


@pytest.mark.parametrize("case", CASES)
def test_many_short_rows_random(L, case):
    """Thousands of rows of a few to a few hundred entries: the 16-lane teams and the
    single-float / pair-access variants of the row kernels."""
    rng = np.random.default_rng(6000 + case)
    n = int(rng.choice([rng.integers(1, 40), rng.integers(1, 12) * 4, rng.integers(1, 40) * 8, rng.integers(40, 300)]))
    G = int(rng.choice([1, 1, 3, 16]))
    w = int(rng.integers(4096 // G + 1, 9000 // G + 2))
    h = G * n
    pad = int(rng.choice([0, 0, 0, 4, 1]))
    tag = f"G={G} n={n} w={w} pad={pad}"
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    # channelwise softmax over G windows of n entries
    cw = L.channelwise_softmax_layer((G, n))
    y = cw.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = cw.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    check("channelwise y " + tag, y, orc.channelwise_softmax_fwd(x, G, n, n), orc.channelwise_softmax_fwd(f64(x), G, n, n))
    check("channelwise dx " + tag, dx, orc.channelwise_softmax_bwd(y, dy, G, n, n),
          orc.channelwise_softmax_bwd(f64(y), f64(dy), G, n, n))
    # layer norm over the same rows, fp32 and fp16 storage, with and without weights
    for half in (False, True):
        affine = bool((case + half) % 2)
        xs, gs = (x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)) if half else (x, dy)
        g = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32) if affine else None
        b = (0.2 * rng.standard_normal(n)).astype(np.float32) if affine else None
        kw = dict(scale_values=g, bias_values=b) if affine else {}
        dims, sd = ((G, n), 1) if G > 1 else ((n,), 0)
        layer = L.layer_norm_layer(dims, 1e-5, affine, affine, sd, **kw)
        tdt, tol = (torch.float16, TOL_F16) if half else (torch.float32, TOL_F32)
        yy = layer.forward(L.DeviceMatrix.from_numpy(xs, dtype=tdt, ldim=h + pad)).to_numpy()
        dd = layer.backward(L.DeviceMatrix.from_numpy(gs, dtype=tdt, ldim=h + pad)).to_numpy()
        ref, ex = {}, {}
        for dst, conv in ((ref, f32), (ex, f64)):
            gg = None if g is None else conv(g)
            bb = None if b is None else conv(b)
            dst["y"], st = orc.layer_norm_fwd(conv(xs), G, n, n, 1e-5, gg, bb)
            dst["dx"], _, dst["dscale"], dst["dbias"] = orc.layer_norm_bwd(conv(xs), conv(gs), st, G, n, n, 1e-5, gg,
                                                                             affine, affine)
        t2 = tag + f" half={half} affine={affine}"
        check("layer norm y " + t2, yy, ref["y"], ex["y"], tol=tol)
        if n > 1:
            check("layer norm dx " + t2, dd, ref["dx"], ex["dx"], tol=tol)
        if affine:
            check("layer norm dscale " + t2, layer.m_scale_gradient.to_numpy(), ref["dscale"], ex["dscale"], tol=tol)
            check("layer norm dbias " + t2, layer.m_bias_gradient.to_numpy(), ref["dbias"], ex["dbias"], tol=tol)


@pytest.mark.parametrize("case", CASES)
def test_small_channels_random(L, case):
    """Batch norm and channel-wise scale/bias on channels of 1 to 70 entries: the row-tile
    kernels (register-resident and three-kernel) next to the channel walk."""
    rng = np.random.default_rng(7000 + case)
    cs = int(rng.choice([1, 1, 2, 4, 8, 9, 16, 25, 49, rng.integers(1, 70)]))
    C = int(rng.integers(1, 600))
    w = int(rng.choice([rng.integers(1, 70), rng.integers(70, 300), rng.integers(300, 700)]))
    h = C * cs
    pad = int(rng.choice([0, 0, 0, 4, 2]))
    bessel = bool(case % 2)
    half = bool(case % 3 == 2)   # fp16 storage: the same kernels with 8-byte row quads
    tag = f"C={C} cs={cs} w={w} pad={pad} half={half}"
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    if half:
        x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (0.1 * rng.standard_normal(C)).astype(np.float32)
    bn = L.batch_normalization_layer((C, cs), 0.9, 1e-5, bessel, g, b)
    tdt = torch.float16 if half else torch.float32
    y = bn.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    dx = bn.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=h + pad)).to_numpy()
    mv = bn.m_mean_and_var.to_numpy()
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        rm, rv = conv(np.zeros(C)), conv(np.ones(C))
        dst["y"], m, v = orc.batch_norm_fwd(conv(x), C, cs, 1e-5, 0.9, conv(g), conv(b), rm, rv, bessel)
        dst["mean"], dst["var"], dst["rmean"], dst["rvar"] = m, v, rm, rv
        dst["dx"], dst["dscale"], dst["dbias"], dst["dmean"], dst["dvar"] = orc.batch_norm_bwd(
            conv(x), conv(dy), C, cs, 1e-5, m, v, conv(g), bessel=bessel)
    mvg = bn.m_mean_and_var_gradient.to_numpy()
    got = dict(y=y, dx=dx, mean=mv[:, 0], var=mv[:, 1], dscale=bn.m_scale_gradient.to_numpy(),
               dbias=bn.m_bias_gradient.to_numpy(), dmean=mvg[:, 0], dvar=mvg[:, 1],
               rmean=bn.weights[2].to_numpy(), rvar=bn.weights[3].to_numpy())
    if cs * w <= 1:
        for k in ("dmean", "dvar", "dscale", "dbias"):
            got.pop(k)
    for k in got:
        check(f"batch norm {k} {tag}", got[k], ref[k], ex[k], tol=TOL_F16 if half and k in ("y", "dx") else TOL_F32)
    wts = np.asfortranarray(np.stack([g, b], axis=1))
    sb = L.channelwise_scale_bias_layer((C, cs))
    sb.set_weights(g, b)
    y = sb.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    dx = sb.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    check("channelwise scale/bias y " + tag, y, orc.channelwise_scale_bias_fwd(x, wts, C, cs),
          orc.channelwise_scale_bias_fwd(f64(x), f64(wts), C, cs))
    rdx, rwg = orc.channelwise_scale_bias_bwd(x, dy, wts, C, cs)
    edx, ewg = orc.channelwise_scale_bias_bwd(f64(x), f64(dy), f64(wts), C, cs)
    check("channelwise scale/bias dx " + tag, dx, rdx, edx)
    check("channelwise scale/bias dweights " + tag, sb.m_weights_gradient.to_numpy(), rwg, ewg)


@pytest.mark.parametrize("case", CASES)
def test_many_long_rows_random(L, case):
    """More long rows than the device holds clusters at once: the persistent cluster kernels
    rotate through several rows per workgroup, and the long-row layer norm streams them."""
    rng = np.random.default_rng(8000 + case)
    n = int(rng.choice([rng.integers(4200, 9000) * 4, rng.integers(9000, 40000) * 4, rng.integers(17000, 150000)]))
    # even cases: at least 48 MiB per tensor, from where the softmax cluster kernels are taken
    w = int(rng.integers(13_000_000 // n + 1, 16_000_000 // n + 2)) if case % 2 == 0 else int(
        rng.integers(2, max(3, 12_000_000 // n)))
    pad = int(rng.choice([0, 0, 4, 1]))
    tag = f"n={n} w={w} pad={pad}"
    x, dy = rand(rng, n, w, 0.0, 2.5), rand(rng, n, w)
    kind, layer, fwd, bwd = (("softmax", L.softmax_layer(), orc.softmax_fwd, orc.softmax_bwd),
                             ("log_softmax", L.log_softmax_layer(), orc.log_softmax_fwd, orc.log_softmax_bwd))[case % 2]
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=n + pad)).to_numpy()
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=n + pad)).to_numpy()
    check(f"{kind} y {tag}", y, fwd(x), fwd(f64(x)))
    check(f"{kind} dx {tag}", dx, bwd(y, dy), bwd(f64(y), f64(dy)))
    half = bool(case % 3 == 1)
    if half:
        x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
    g = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    b = (0.2 * rng.standard_normal(n)).astype(np.float32)
    ln = L.layer_norm_layer((n,), 1e-5, True, True, 0, scale_values=g, bias_values=b)
    tdt, tol = (torch.float16, TOL_F16) if half else (torch.float32, TOL_F32)
    y = ln.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=n + pad)).to_numpy()
    dx = ln.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=n + pad)).to_numpy()
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        dst["y"], st = orc.layer_norm_fwd(conv(x), 1, n, n, 1e-5, conv(g), conv(b))
        dst["dx"], _, dst["dscale"], dst["dbias"] = orc.layer_norm_bwd(conv(x), conv(dy), st, 1, n, n, 1e-5, conv(g),
                                                                         True, True)
    check(f"layer norm y {tag} half={half}", y, ref["y"], ex["y"], tol=tol)
    check(f"layer norm dx {tag} half={half}", dx, ref["dx"], ex["dx"], tol=tol)
    check(f"layer norm dscale {tag} half={half}", ln.m_scale_gradient.to_numpy(), ref["dscale"], ex["dscale"], tol=tol)
    check(f"layer norm dbias {tag} half={half}", ln.m_bias_gradient.to_numpy(), ref["dbias"], ex["dbias"], tol=tol)


@pytest.mark.parametrize("case", CASES)
def test_many_large_channels_random(L, case):
    """Batch norm with more channels than resident clusters (fp32 and fp16 storage) and channel
    sizes from a few vectors to a few thousand."""
    rng = np.random.default_rng(9000 + case)
    cs = int(rng.choice([8, 12, 16, 24, 32, 64, 196, 784, rng.integers(3, 200) * 8]))
    w = int(rng.choice([rng.integers(2, 40), rng.integers(40, 400), rng.integers(400, 1200)]))
    C = int(max(2, min(3000, rng.integers(4_000_000, 16_000_000) // (cs * w))))
    h = C * cs
    pad = int(rng.choice([0, 0, 8, 4]))
    half = bool(case % 3 == 2)
    bessel = bool(case % 2)
    tag = f"C={C} cs={cs} w={w} pad={pad} half={half}"
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    if half:
        x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (0.1 * rng.standard_normal(C)).astype(np.float32)
    bn = L.batch_normalization_layer((C, cs), 0.9, 1e-5, bessel, g, b)
    tdt, tol = (torch.float16, TOL_F16) if half else (torch.float32, TOL_F32)
    y = bn.forward(L.DeviceMatrix.from_numpy(x, dtype=tdt, ldim=h + pad)).to_numpy()
    dx = bn.backward(L.DeviceMatrix.from_numpy(dy, dtype=tdt, ldim=h + pad)).to_numpy()
    mv, mvg = bn.m_mean_and_var.to_numpy(), bn.m_mean_and_var_gradient.to_numpy()
    ref, ex = {}, {}
    for dst, conv in ((ref, f32), (ex, f64)):
        rm, rv = conv(np.zeros(C)), conv(np.ones(C))
        dst["y"], m, v = orc.batch_norm_fwd(conv(x), C, cs, 1e-5, 0.9, conv(g), conv(b), rm, rv, bessel)
        dst["mean"], dst["var"] = m, v
        dst["dx"], dst["dscale"], dst["dbias"], dst["dmean"], dst["dvar"] = orc.batch_norm_bwd(
            conv(x), conv(dy), C, cs, 1e-5, m, v, conv(g), bessel=bessel)
    got = dict(y=y, dx=dx, mean=mv[:, 0], var=mv[:, 1], dscale=bn.m_scale_gradient.to_numpy(),
               dbias=bn.m_bias_gradient.to_numpy(), dmean=mvg[:, 0], dvar=mvg[:, 1])
    for k in got:
        # statistics and their gradients are fp32 whatever the storage type
        check(f"batch norm {k} {tag}", got[k], ref[k], ex[k], tol=tol if k in ("y", "dx") else TOL_F32)
