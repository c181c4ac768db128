"""The header-only C++ adapter (lbann_amd/adapter/lbnorm_layers.hpp) through its test
driver: host-side behaviour on the CPU, numerical parity with the oracle on the GPU."""
import ctypes
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "cpp", "libadapter_driver.so")

i64, vp, cint, dbl = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_double


def driver():
    assert os.path.exists(DRIVER), "build it with `python -m lbann_amd.build`"
    # torch first: it brings its own HIP runtime, and the driver must bind to that one
    # rather than pull a second runtime into the process
    import torch  # noqa: F401
    return ctypes.CDLL(DRIVER)


def test_adapter_host_logic_and_errors():
    """Dimension logic and the reference's error cases (bad softmax mode, bad start_dim,
    bad channelwise dim, non-local batch-norm statistics) without touching a device."""
    assert driver().drv_error_cases() == 0


def _dims(d):
    return (i64 * len(d))(*d), len(d)


@pytest.mark.gpu
def test_adapter_layers_match_oracle():
    import torch
    from oracle import cpu_oracle as orc
    from tests.parity import TOL_F16, check
    from lbann_amd.layers import DeviceMatrix
    d = driver()
    err = ctypes.create_string_buffer(512)
    st = vp(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(3)
    mk = lambda h, w, m=0.0, s=1.0: np.asfortranarray((rng.standard_normal((w, h)) * s + m).astype(np.float32).T)
    dev = lambda a: torch.from_numpy(np.asarray(a, np.float32)).cuda()
    p = lambda t: vp(t.data_ptr())

    # ---- layer norm, start_dim = -1 on (6, 512) samples, affine, fp32 and fp16 storage
    dims, w = (6, 512), 20
    h = 6 * 512
    g = (1 + 0.2 * rng.standard_normal(512)).astype(np.float32)
    b = (0.2 * rng.standard_normal(512)).astype(np.float32)
    for half in (0, 1):
        x, dy = mk(h, w, 0.3, 1.5), mk(h, w)
        if half:
            x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
        tdt = torch.float16 if half else torch.float32
        mx, mdy = DeviceMatrix.from_numpy(x, dtype=tdt), DeviceMatrix.from_numpy(dy, dtype=tdt)
        my, mdx = DeviceMatrix(h, w, dtype=tdt), DeviceMatrix(h, w, dtype=tdt)
        gw, bw, dg, db = dev(g), dev(b), torch.empty(512).cuda(), torch.empty(512).cuda()
        stats, sgrad = DeviceMatrix(12, w), DeviceMatrix(12, w)
        da, nd = _dims(dims)
        rc = d.drv_layer_norm(cint(half), da, cint(nd), cint(-1), cint(1), cint(1), dbl(1e-5), i64(h), i64(w), i64(h),
                              mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(gw), p(bw), p(dg), p(db),
                              stats.Buffer(), sgrad.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        y_ref, st_ref = orc.layer_norm_fwd(x, 6, 512, 512, 1e-5, g, b)
        dx_ref, sg_ref, dg_ref, db_ref = orc.layer_norm_bwd(x, dy, st_ref, 6, 512, 512, 1e-5, g, True, True)
        tol = TOL_F16 if half else 1e-5
        check("adapter ln y", my.to_numpy(), y_ref, tol=tol)
        check("adapter ln dx", mdx.to_numpy(), dx_ref, tol=tol)
        check("adapter ln stats", stats.to_numpy(), st_ref, tol=tol)
        check("adapter ln sgrad", sgrad.to_numpy(), sg_ref, tol=tol)
        check("adapter ln dscale", dg.cpu().numpy(), dg_ref, tol=tol)
        check("adapter ln dbias", db.cpu().numpy(), db_ref, tol=tol)

    # ---- batch norm (8, 12, 12) x 10, fp32 and fp16 storage
    dims, w = (8, 12, 12), 10
    h = 8 * 144
    g = rng.uniform(0.5, 1.5, 8).astype(np.float32)
    b = (0.1 * rng.standard_normal(8)).astype(np.float32)
    for half in (0, 1):
        x, dy = mk(h, w, 2.0, 3.0), mk(h, w)
        if half:
            x, dy = x.astype(np.float16).astype(np.float32), dy.astype(np.float16).astype(np.float32)
        tdt = torch.float16 if half else torch.float32
        tol = TOL_F16 if half else 1e-5
        mx, mdy = DeviceMatrix.from_numpy(x, dtype=tdt), DeviceMatrix.from_numpy(dy, dtype=tdt)
        my, mdx = DeviceMatrix(h, w, dtype=tdt), DeviceMatrix(h, w, dtype=tdt)
        gw, bw, rm, rv = dev(g), dev(b), torch.zeros(8).cuda(), torch.ones(8).cuda()
        dg, db = torch.empty(8).cuda(), torch.empty(8).cuda()
        mv, mvg = DeviceMatrix(8, 2), DeviceMatrix(8, 2)
        da, nd = _dims(dims)
        rc = d.drv_batch_norm(cint(half), da, cint(nd), dbl(0.9), dbl(1e-5), cint(1), cint(1), i64(h), i64(w),
                              i64(h), mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(gw), p(bw), p(rm),
                              p(rv), p(dg), p(db), mv.Buffer(), mvg.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        rm0, rv0 = np.zeros(8, np.float32), np.ones(8, np.float32)
        y_ref, m_ref, v_ref = orc.batch_norm_fwd(x, 8, 144, 1e-5, 0.9, g, b, rm0, rv0)
        dx_ref, dg_ref, db_ref, dm_ref, dv_ref = orc.batch_norm_bwd(x, dy, 8, 144, 1e-5, m_ref, v_ref, g)
        check("adapter bn y", my.to_numpy(), y_ref, tol=tol)
        check("adapter bn dx", mdx.to_numpy(), dx_ref, tol=tol)
        check("adapter bn mean/var", mv.to_numpy(), np.stack([m_ref, v_ref], axis=1), tol=tol)
        check("adapter bn dmean/dvar", mvg.to_numpy(), np.stack([dm_ref, dv_ref], axis=1), tol=tol)
        check("adapter bn dscale", dg.cpu().numpy(), dg_ref, tol=tol)
        check("adapter bn dbias", db.cpu().numpy(), db_ref, tol=tol)
        check("adapter bn running mean", rm.cpu().numpy(), rm0, tol=tol)
        check("adapter bn running var", rv.cpu().numpy(), rv0, tol=tol)

    # ---- softmax family, incl. a row long enough for the split kernels (workspace path)
    for kind, h, w, dims, dim, single in ((0, 4096, 9, (4096,), 0, 0), (1, 1000, 7, (1000,), 0, 0),
                                          (0, 70000, 2, (70000,), 0, 0), (2, 5 * 2 * 8, 11, (5, 2, 8), -1, 1),
                                          (2, 16 * 256, 6, (16, 256), 0, 0)):
        x, dy = mk(h, w, 0.0, 2.0), mk(h, w)
        mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w), DeviceMatrix(h, w)
        da, nd = _dims(dims)
        rc = d.drv_softmax_family(cint(kind), da, cint(nd), i64(dim), cint(single), i64(h), i64(w), i64(h),
                                  mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        if kind == 0:
            fwd, bwd = orc.softmax_fwd, orc.softmax_bwd
        elif kind == 1:
            fwd, bwd = orc.log_softmax_fwd, orc.log_softmax_bwd
        else:
            cs = dims[-1] if single else h // dims[0]
            C = h // cs
            fwd = lambda a: orc.channelwise_softmax_fwd(a, C, cs, cs)
            bwd = lambda yy, gg: orc.channelwise_softmax_bwd(yy, gg, C, cs, cs)
        f64 = lambda a: np.asfortranarray(np.asarray(a, np.float64))
        y = my.to_numpy()
        check(f"adapter softmax kind {kind} y", y, fwd(x), fwd(f64(x)))
        check(f"adapter softmax kind {kind} dx", mdx.to_numpy(), bwd(y, dy), bwd(f64(y), f64(dy)))

    # ---- softmax and log-softmax on fp16 storage: a matrix type with 2-byte elements
    import torch as _torch
    h, w = 4096, 12
    x16 = mk(h, w, 0.0, 2.0).astype(np.float16)
    dy16 = mk(h, w).astype(np.float16)
    xf, dyf = np.asfortranarray(x16.astype(np.float32)), np.asfortranarray(dy16.astype(np.float32))
    for kind in (0, 1):
        mx = DeviceMatrix.from_numpy(x16, dtype=_torch.float16)
        mdy = DeviceMatrix.from_numpy(dy16, dtype=_torch.float16)
        my, mdx = DeviceMatrix(h, w, dtype=_torch.float16), DeviceMatrix(h, w, dtype=_torch.float16)
        rc = d.drv_softmax_family_f16(cint(kind), i64(h), i64(w), i64(h), mx.Buffer(), my.Buffer(), mdy.Buffer(),
                                      mdx.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        fwd, bwd = (orc.softmax_fwd, orc.softmax_bwd) if kind == 0 else (orc.log_softmax_fwd, orc.log_softmax_bwd)
        y = my.to_numpy()
        check(f"adapter f16 softmax kind {kind} y", y, fwd(xf), tol=TOL_F16)
        check(f"adapter f16 softmax kind {kind} dx", mdx.to_numpy(), bwd(np.asfortranarray(y), dyf), tol=TOL_F16)

    # ---- cross entropy with fp16 storage
    h, w = 520, 9
    x16 = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float16).T)
    t16 = np.asfortranarray(rng.uniform(-0.3, 1.0, (w, h)).astype(np.float16).T)
    g16 = rng.standard_normal(w).astype(np.float16)
    half = _torch.float16
    mx, mt = DeviceMatrix.from_numpy(x16, dtype=half), DeviceMatrix.from_numpy(t16, dtype=half)
    mdl = DeviceMatrix.from_numpy(np.asfortranarray(g16.reshape(1, w)), dtype=half)
    ml, mdx, mdt = DeviceMatrix(1, w, dtype=half), DeviceMatrix(h, w, dtype=half), DeviceMatrix(h, w, dtype=half)
    da, nd = _dims((h,))
    rc = d.drv_cross_entropy_f16(da, cint(nd), i64(h), i64(w), mx.Buffer(), mt.Buffer(), ml.Buffer(), mdl.Buffer(),
                                 mdx.Buffer(), mdt.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    xf, tf, gf = (np.asfortranarray(a.astype(np.float32)) for a in (x16, t16, g16))
    check("adapter f16 cross entropy loss", ml.to_numpy()[0].astype(np.float32), orc.cross_entropy_fwd(xf, tf), tol=TOL_F16)
    dx_ref, dt_ref = orc.cross_entropy_bwd(xf, tf, gf)
    check("adapter f16 cross entropy dx", mdx.to_numpy().astype(np.float32), dx_ref, tol=TOL_F16)
    check("adapter f16 cross entropy dtruth", mdt.to_numpy().astype(np.float32), dt_ref, tol=TOL_F16)

    # ---- instance norm on (6, 20, 20) samples
    dims, w = (6, 20, 20), 9
    h = 6 * 400
    x, dy = mk(h, w, 0.5, 2.0), mk(h, w)
    mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w), DeviceMatrix(h, w)
    da, nd = _dims(dims)
    rc = d.drv_instance_norm(da, cint(nd), dbl(1e-5), i64(h), i64(w), i64(h), mx.Buffer(), my.Buffer(),
                             mdy.Buffer(), mdx.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    y_ref, sums = orc.instance_norm_fwd(x, 6, 400, 1e-5)
    check("adapter instance norm y", my.to_numpy(), y_ref)
    check("adapter instance norm dx", mdx.to_numpy(), orc.instance_norm_bwd(x, dy, sums, 6, 400, 1e-5))

    # ---- entry-wise batch norm on (4, 40) samples, 12 per mini-batch
    dims, w = (4, 40), 12
    h = 160
    x, dy = mk(h, w, 0.5, 2.0), mk(h, w)
    mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w), DeviceMatrix(h, w)
    rm, rv = torch.zeros(h).cuda(), torch.ones(h).cuda()
    stats, sgrad = DeviceMatrix(h, 2), DeviceMatrix(h, 2)
    da, nd = _dims(dims)
    rc = d.drv_entrywise_batch_norm(da, cint(nd), dbl(0.9), dbl(1e-5), cint(1), i64(h), i64(w), i64(h), mx.Buffer(),
                                    my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(rm), p(rv), stats.Buffer(),
                                    sgrad.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    rm0, rv0 = np.zeros(h, np.float32), np.ones(h, np.float32)
    y_ref, st_ref = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, rm0, rv0)
    dx_ref, sg_ref = orc.entrywise_batch_norm_bwd(x, dy, st_ref, 1e-5)
    check("adapter entrywise bn y", my.to_numpy(), y_ref)
    check("adapter entrywise bn dx", mdx.to_numpy(), dx_ref)
    check("adapter entrywise bn stats", stats.to_numpy(), st_ref)
    check("adapter entrywise bn stats grad", sgrad.to_numpy(), sg_ref)
    check("adapter entrywise bn running mean", rm.cpu().numpy(), rm0)
    check("adapter entrywise bn running var", rv.cpu().numpy(), rv0)

    # ---- cross entropy on (3, 8, 8) predictions: dense ground truth and labels
    h, sp, w = 192, 64, 12
    x = np.asfortranarray(rng.uniform(0.25, 1.0, (w, h)).astype(np.float32).T)
    dense = np.asfortranarray(rng.uniform(-0.2, 1.0, (w, h)).astype(np.float32).T)
    labels = np.asfortranarray(rng.integers(0, 3, (w, sp)).astype(np.float32).T)
    dloss = rng.standard_normal(w).astype(np.float32)
    for use_labels, truth, tdims in ((0, dense, (3, 8, 8)), (1, labels, (1, 8, 8))):
        mx, mt = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(truth)
        ml, mdl = DeviceMatrix(1, w), DeviceMatrix.from_numpy(dloss.reshape(1, -1))
        mdx, mdt = DeviceMatrix(h, w), DeviceMatrix(truth.shape[0], w, fill=7.0)
        pa, nd = _dims((3, 8, 8))
        ta, _ = _dims(tdims)
        rc = d.drv_cross_entropy(pa, ta, cint(nd), cint(use_labels), i64(h), i64(truth.shape[0]), i64(w), mx.Buffer(),
                                 mt.Buffer(), ml.Buffer(), mdl.Buffer(), mdx.Buffer(), mdt.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        check("adapter cross entropy loss", ml.to_numpy()[0], orc.cross_entropy_fwd(x, truth, bool(use_labels)))
        dx_ref, dt_ref = orc.cross_entropy_bwd(x, truth, dloss, bool(use_labels))
        check("adapter cross entropy dx", mdx.to_numpy(), dx_ref)
        if use_labels:
            assert np.all(mdt.to_numpy() == 7.0)   # untouched, as in the reference
        else:
            check("adapter cross entropy dtruth", mdt.to_numpy(), dt_ref)

    # ---- softmax -> cross entropy through the fused forward: (1000,) dense (one kernel), (3, 8, 8) labels (two)
    for use_labels, pdims, tdims in ((0, (1000,), (1000,)), (1, (3, 8, 8), (1, 8, 8))):
        h, w = int(np.prod(pdims)), 20
        x = mk(h, w, 0.0, 2.0)
        if use_labels:
            truth = np.asfortranarray(rng.integers(0, 3, (w, 64)).astype(np.float32).T)
        else:
            truth = np.asfortranarray(rng.uniform(-0.2, 1.0, (w, h)).astype(np.float32).T)
        dloss = rng.standard_normal(w).astype(np.float32)
        mx, my, mt = DeviceMatrix.from_numpy(x), DeviceMatrix(h, w), DeviceMatrix.from_numpy(truth)
        ml, mdl = DeviceMatrix(1, w), DeviceMatrix.from_numpy(dloss.reshape(1, -1))
        mdy, mdx, mdt = DeviceMatrix(h, w), DeviceMatrix(h, w), DeviceMatrix(truth.shape[0], w)
        pa, nd = _dims(pdims)
        ta, _ = _dims(tdims)
        for fused_bwd in (0, 1):
            mdy.tensor.fill_(-3.0)
            rc = d.drv_softmax_cross_entropy(pa, ta, cint(nd), cint(use_labels), i64(h), i64(truth.shape[0]), i64(w),
                                             mx.Buffer(), my.Buffer(), mt.Buffer(), ml.Buffer(), mdl.Buffer(),
                                             mdy.Buffer(), mdx.Buffer(), mdt.Buffer(), cint(fused_bwd), st, err, cint(512))
            assert rc == 0, err.value
            y_ref = orc.softmax_fwd(x)
            check("adapter softmax+ce y", my.to_numpy(), y_ref)
            check("adapter softmax+ce loss", ml.to_numpy()[0], orc.cross_entropy_fwd(y_ref, truth, bool(use_labels)))
            dp_ref, dt_ref = orc.cross_entropy_bwd(y_ref, truth, dloss, bool(use_labels))
            if fused_bwd:
                assert torch.all(mdy.tensor == -3.0).item()   # the gradient w.r.t. the prediction is never written
            else:
                check("adapter softmax+ce dprediction", mdy.to_numpy(), dp_ref)
            check("adapter softmax+ce dx", mdx.to_numpy(), orc.softmax_bwd(y_ref, dp_ref))
            if not use_labels:
                check("adapter softmax+ce dtruth", mdt.to_numpy(), dt_ref)

    # ---- scale/bias layers on (8, 12, 12) x 10
    dims, w = (8, 12, 12), 10
    h = 8 * 144
    x, dy = mk(h, w, 0.5, 2.0), mk(h, w)
    for kind, n in ((0, h), (1, 8)):
        wts = np.asfortranarray(np.stack([rng.normal(1, 1, n), rng.normal(0, 1, n)], axis=1).astype(np.float32))
        mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w), DeviceMatrix(h, w)
        mw, mwg = DeviceMatrix.from_numpy(wts), DeviceMatrix(n, 2)
        da, nd = _dims(dims)
        rc = d.drv_scale_bias(cint(kind), da, cint(nd), i64(h), i64(w), i64(h), mx.Buffer(), my.Buffer(), mdy.Buffer(),
                              mdx.Buffer(), mw.Buffer(), i64(n), mwg.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        if kind == 0:
            y_ref = orc.entrywise_scale_bias_fwd(x, wts)
            dx_ref, wg_ref = orc.entrywise_scale_bias_bwd(x, dy, wts)
        else:
            y_ref = orc.channelwise_scale_bias_fwd(x, wts, 8, 144)
            dx_ref, wg_ref = orc.channelwise_scale_bias_bwd(x, dy, wts, 8, 144)
        check(f"adapter scale/bias {kind} y", my.to_numpy(), y_ref)
        check(f"adapter scale/bias {kind} dx", mdx.to_numpy(), dx_ref)
        check(f"adapter scale/bias {kind} dweights", mwg.to_numpy(), wg_ref)

    # ---- channel-wise scale/bias weight gradients into a gradient buffer, twice
    wts = np.asfortranarray(np.stack([rng.normal(1, 1, 8), rng.normal(0, 1, 8)], axis=1).astype(np.float32))
    mx, mdy, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w)
    mw, grad = DeviceMatrix.from_numpy(wts), DeviceMatrix(8, 2, ldim=12, fill=float("nan"))
    statuses = (ctypes.c_int * 2)()
    da, nd = _dims(dims)
    rc = d.drv_gradient_buffer(da, cint(nd), i64(h), i64(w), mx.Buffer(), mdy.Buffer(), mdx.Buffer(), mw.Buffer(),
                               grad.Buffer(), i64(12), ctypes.c_float(0.5), ctypes.c_float(-2.0), statuses, st, err,
                               cint(512))
    assert rc == 0, err.value
    assert list(statuses) == [0, 2]          # ready after the first contribution, sync_needed after the second
    _, wg_ref = orc.channelwise_scale_bias_bwd(x, dy, wts, 8, 144)
    wg_dev = None
    # the buffer holds Scale + Axpy of the device's own weight gradient, to the bit
    mwg = DeviceMatrix(8, 2)
    rc = d.drv_scale_bias(cint(1), da, cint(nd), i64(h), i64(w), i64(h), mx.Buffer(), DeviceMatrix(h, w).Buffer(),
                          mdy.Buffer(), mdx.Buffer(), mw.Buffer(), i64(8), mwg.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    wg_dev = mwg.to_numpy()
    exp = orc.gradient_sink(orc.gradient_sink(np.zeros((8, 2), np.float32), wg_dev, 0.0, 0.5), wg_dev, 1.0, -2.0)
    assert grad.to_numpy().tobytes() == exp.tobytes()
    check("adapter gradient buffer", grad.to_numpy(), -1.5 * wg_ref)
    assert torch.isnan(grad.tensor[:, 8:]).all()

    # ---- entry-wise batch norm with the mini-batch on two ranks (all-reduce hook of the adapter)
    dims, w, w0 = (5, 8, 6), 27, 11
    h = 240
    x, dy = mk(h, w, -0.4, 1.7), mk(h, w)
    mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), DeviceMatrix(h, w), DeviceMatrix(h, w)
    rm2 = torch.zeros(2 * h, device="cuda")
    rv2 = torch.ones(2 * h, device="cuda")
    stats = DeviceMatrix(h, 2)
    da, nd = _dims(dims)
    rc = d.drv_entrywise_batch_norm_two_ranks(da, cint(nd), dbl(0.9), dbl(1e-5), i64(h), i64(w), i64(w0), i64(h), mx.Buffer(),
                                              my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(rm2), p(rv2), stats.Buffer(), st, err,
                                              cint(512))
    assert rc == 0, err.value
    rm0, rv0 = np.zeros(h, np.float32), np.ones(h, np.float32)
    y_ref, st_ref = orc.entrywise_batch_norm_fwd(x, 0.9, 1e-5, rm0, rv0)
    dx_ref, _ = orc.entrywise_batch_norm_bwd(x, dy, st_ref, 1e-5)
    x64, dy64 = x.astype(np.float64, order="F"), dy.astype(np.float64, order="F")
    y64, st64 = orc.entrywise_batch_norm_fwd(x64, 0.9, 1e-5, np.zeros(h), np.ones(h))
    dx64, _ = orc.entrywise_batch_norm_bwd(x64, dy64, st64, 1e-5)
    check("adapter two-rank entrywise bn y", my.to_numpy(), y_ref, y64)
    check("adapter two-rank entrywise bn dx", mdx.to_numpy(), dx_ref, dx64)
    check("adapter two-rank entrywise bn stats", stats.to_numpy(), st_ref, st64)
    for k in range(2):
        check("adapter two-rank running mean", rm2[k * h:(k + 1) * h].cpu().numpy(), rm0)
        check("adapter two-rank running var", rv2[k * h:(k + 1) * h].cpu().numpy(), rv0)


@pytest.mark.gpu
def test_adapter_layers_of_doubles_match_oracle():
    """TensorDataType = double through the C++ adapter: layer_norm_layer<double>,
    batch_normalization_layer<double> and the softmax family on device_matrix<double>."""
    import torch
    from oracle import cpu_oracle as orc
    from tests.parity import TOL_F64, check
    from lbann_amd.layers import DeviceMatrix
    d = driver()
    err = ctypes.create_string_buffer(512)
    st = vp(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(31)
    F64 = torch.float64
    mk = lambda h, w, m=0.0, s=1.0: np.asfortranarray((rng.standard_normal((w, h)) * s + m).T)
    dev = lambda a: torch.from_numpy(np.asarray(a, np.float64)).cuda()
    p = lambda t: vp(t.data_ptr())
    new = lambda h, w: DeviceMatrix(h, w, dtype=F64)

    dims, w = (6, 512), 20
    h = 6 * 512
    g, b = 1 + 0.2 * rng.standard_normal(512), 0.2 * rng.standard_normal(512)
    x, dy = mk(h, w, 0.3, 1.5), mk(h, w)
    mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), new(h, w), new(h, w)
    gw, bw = dev(g), dev(b)
    dg, db = torch.empty(512, dtype=F64).cuda(), torch.empty(512, dtype=F64).cuda()
    stats, sgrad = new(12, w), new(12, w)
    da, nd = _dims(dims)
    rc = d.drv_layer_norm(cint(2), da, cint(nd), cint(-1), cint(1), cint(1), dbl(1e-5), i64(h), i64(w), i64(h),
                          mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(gw), p(bw), p(dg), p(db),
                          stats.Buffer(), sgrad.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    y_ref, st_ref = orc.layer_norm_fwd(x, 6, 512, 512, 1e-5, g, b)
    dx_ref, sg_ref, dg_ref, db_ref = orc.layer_norm_bwd(x, dy, st_ref, 6, 512, 512, 1e-5, g, True, True)
    for name, got, ref in (("y", my.to_numpy(), y_ref), ("dx", mdx.to_numpy(), dx_ref), ("stats", stats.to_numpy(), st_ref),
                           ("sgrad", sgrad.to_numpy(), sg_ref), ("dscale", dg.cpu().numpy(), dg_ref),
                           ("dbias", db.cpu().numpy(), db_ref)):
        assert got.dtype == np.float64
        check(f"adapter f64 ln {name}", got, ref, tol=TOL_F64)

    dims, w = (8, 12, 12), 10
    h = 8 * 144
    g, b = rng.uniform(0.5, 1.5, 8), 0.1 * rng.standard_normal(8)
    x, dy = mk(h, w, 2.0, 3.0), mk(h, w)
    mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), new(h, w), new(h, w)
    gw, bw, rm, rv = dev(g), dev(b), torch.zeros(8, dtype=F64).cuda(), torch.ones(8, dtype=F64).cuda()
    dg, db = torch.empty(8, dtype=F64).cuda(), torch.empty(8, dtype=F64).cuda()
    mv, mvg = new(8, 2), new(8, 2)
    da, nd = _dims(dims)
    rc = d.drv_batch_norm(cint(2), da, cint(nd), dbl(0.9), dbl(1e-5), cint(1), cint(1), i64(h), i64(w),
                          i64(h), mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), p(gw), p(bw), p(rm),
                          p(rv), p(dg), p(db), mv.Buffer(), mvg.Buffer(), st, err, cint(512))
    assert rc == 0, err.value
    rm0, rv0 = np.zeros(8), np.ones(8)
    y_ref, m_ref, v_ref = orc.batch_norm_fwd(x, 8, 144, 1e-5, 0.9, g, b, rm0, rv0)
    dx_ref, dg_ref, db_ref, dm_ref, dv_ref = orc.batch_norm_bwd(x, dy, 8, 144, 1e-5, m_ref, v_ref, g)
    for name, got, ref in (("y", my.to_numpy(), y_ref), ("dx", mdx.to_numpy(), dx_ref),
                           ("mean/var", mv.to_numpy(), np.stack([m_ref, v_ref], axis=1)),
                           ("dmean/dvar", mvg.to_numpy(), np.stack([dm_ref, dv_ref], axis=1)),
                           ("dscale", dg.cpu().numpy(), dg_ref), ("dbias", db.cpu().numpy(), db_ref),
                           ("running mean", rm.cpu().numpy(), rm0), ("running var", rv.cpu().numpy(), rv0)):
        check(f"adapter f64 bn {name}", got, ref, tol=TOL_F64)

    for kind, h, w, dims, dim, single in ((0, 4096, 9, (4096,), 0, 0), (1, 1000, 7, (1000,), 0, 0),
                                          (0, 70000, 2, (70000,), 0, 0), (2, 5 * 2 * 8, 11, (5, 2, 8), -1, 1),
                                          (2, 16 * 256, 6, (16, 256), 0, 0)):
        x, dy = mk(h, w, 0.0, 2.0), mk(h, w)
        mx, mdy, my, mdx = DeviceMatrix.from_numpy(x), DeviceMatrix.from_numpy(dy), new(h, w), new(h, w)
        da, nd = _dims(dims)
        rc = d.drv_softmax_family_f64(cint(kind), da, cint(nd), i64(dim), cint(single), i64(h), i64(w), i64(h),
                                      mx.Buffer(), my.Buffer(), mdy.Buffer(), mdx.Buffer(), st, err, cint(512))
        assert rc == 0, err.value
        if kind == 0:
            fwd, bwd = orc.softmax_fwd, orc.softmax_bwd
        elif kind == 1:
            fwd, bwd = orc.log_softmax_fwd, orc.log_softmax_bwd
        else:
            cs = dims[-1] if single else h // dims[0]
            C = h // cs
            fwd = lambda a: orc.channelwise_softmax_fwd(a, C, cs, cs)
            bwd = lambda yy, gg: orc.channelwise_softmax_bwd(yy, gg, C, cs, cs)
        y = my.to_numpy()
        check(f"adapter f64 softmax kind {kind} y", y, fwd(x), tol=TOL_F64)
        check(f"adapter f64 softmax kind {kind} dx", mdx.to_numpy(), bwd(y, dy), tol=TOL_F64)
