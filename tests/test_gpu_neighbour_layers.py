"""GPU parity of the layers either side of the normalization / softmax path: cross
entropy (consumes the softmax output) and the entry-wise / channel-wise scale-bias
layers (the learned affine after a normalization layer), through the C ABI against
the CPU oracle.  Tolerance 1e-5 (tests/parity.py), with the float64 oracle as the
tie-breaker where the fp32 reference is itself noisier than that.
"""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import TOL_F16, TOL_F32, check, rel_err

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


def vec_to_row(L, v):
    return L.DeviceMatrix.from_numpy(np.asarray(v, np.float32).reshape(1, -1))


# ===================================================================== cross entropy
CE_DENSE = [
    # (h, w, ld_pad)
    (10, 128, 0), (1000, 64, 0), (192, 23, 0), (4096, 33, 0), (7, 5, 0), (1001, 3, 0), (130, 4, 2),
    (512, 9, 64), (300000, 3, 0), (1 << 20, 2, 0), (65536, 40, 0), (1, 6, 0),
    (16384, 256, 0), (4101, 257, 0),   # one 1024-thread workgroup per column, vector and scalar
    (10, 5000, 0), (21, 70000, 0), (64, 4099, 3), (1, 6000, 0), (3, 100000, 0), (17, 4096, 0),   # 16-lane teams
    (2000000, 1, 0), (600000, 2, 0),   # a column or two: many workgroups per column
    # columns off the 16-byte grid: unaligned vectors and the h % 4 entries behind them
    (17, 40, 0), (19, 300, 0), (1003, 70, 0), (50257, 5, 0), (2048, 9, 1), (4099, 300, 2), (600001, 2, 0), (16, 33, 3),
]


@pytest.mark.parametrize("h,w,pad", CE_DENSE)
def test_cross_entropy_dense(L, h, w, pad):
    rng = np.random.default_rng(h * 7 + w)
    x = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float32).T)
    truth = np.asfortranarray(rng.uniform(-0.3, 1.0, (w, h)).astype(np.float32).T)  # a quarter <= 0: skipped
    truth[0, :] = 0.0
    dy = rng.standard_normal(w).astype(np.float32)
    layer = L.cross_entropy_layer((h,))
    ld = h + pad
    loss = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=ld), L.DeviceMatrix.from_numpy(truth, ldim=ld)).to_numpy()
    check(f"cross entropy loss {h}x{w}", loss[0], orc.cross_entropy_fwd(x, truth), orc.cross_entropy_fwd(f64(x), f64(truth)))
    dx, dt = layer.backward(vec_to_row(L, dy))
    rx, rt = orc.cross_entropy_bwd(x, truth, dy)
    ex, et = orc.cross_entropy_bwd(f64(x), f64(truth), dy.astype(np.float64))
    got = dx.to_numpy()
    check(f"cross entropy dx {h}x{w}", got, rx, ex)
    assert np.all(got[truth <= 0] == 0.0)
    check(f"cross entropy dtruth {h}x{w}", dt.to_numpy(), rt, et)


CE_LABELS = [
    # (classes, spatial dims, w, ld_pad)
    (3, (8, 8), 23, 0), (3, (4, 4, 4), 11, 0), (10, (1,), 64, 0), (5, (7, 3), 9, 0), (4, (6,), 5, 3),
    (21, (64, 64), 6, 0), (2, (300, 300), 3, 0), (1000, (1,), 128, 0), (19, (128, 130), 2, 0),
    (19, (512, 1024), 1, 0),   # one column of a large map: many workgroups per column
    (1000, (1,), 300, 0), (1003, (1,), 70, 3), (17, (1,), 5000, 1), (50257, (1,), 9, 0),   # one label per sample
]


@pytest.mark.parametrize("classes,spatial,w,pad", CE_LABELS)
def test_cross_entropy_labels(L, classes, spatial, w, pad):
    rng = np.random.default_rng(classes * 100 + w)
    sp = int(np.prod(spatial))
    h = classes * sp
    x = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float32).T)
    labels = np.asfortranarray(rng.integers(0, classes, (w, sp)).astype(np.float32).T)
    if sp > 2:
        labels[1, 0] = classes      # a label no class matches contributes nothing
        labels[2, 0] = -3.0
    elif w > 3:
        labels[0, 1] = classes
        labels[0, 2] = -3.0
    dy = rng.standard_normal(w).astype(np.float32)
    layer = L.cross_entropy_layer((classes,) + tuple(spatial), use_labels=True)
    loss = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad),
                         L.DeviceMatrix.from_numpy(labels, ldim=sp + pad)).to_numpy()
    check(f"cross entropy (labels) loss {classes}x{sp}x{w}", loss[0], orc.cross_entropy_fwd(x, labels, True),
          orc.cross_entropy_fwd(f64(x), f64(labels), True))
    dx, none = layer.backward(vec_to_row(L, dy))
    assert none is None
    check(f"cross entropy (labels) dx {classes}x{sp}x{w}", dx.to_numpy(), orc.cross_entropy_bwd(x, labels, dy, True)[0],
          orc.cross_entropy_bwd(f64(x), f64(labels), dy.astype(np.float64), True)[0])


CE_F16 = [
    # (h, w, ld_pad): whole 16-byte vectors of 8, ragged heights, a padded leading dimension, 1024-thread columns
    (16, 128, 0), (1000, 64, 0), (192, 23, 0), (4096, 33, 0), (7, 5, 0), (1001, 3, 0), (136, 4, 8), (130, 4, 2),
    (16384, 256, 0), (4101, 257, 0), (65536, 40, 0), (300000, 3, 0), (1, 6, 0),
    (10, 5000, 0), (33, 4500, 8), (64, 4100, 0),   # 16-lane teams
    # columns off the 16-byte grid: unaligned vectors and the h % 8 entries behind them
    (33, 40, 0), (39, 300, 0), (1003, 70, 0), (50257, 5, 0), (2048, 9, 1), (4103, 300, 2), (600001, 2, 0), (32, 33, 3),
]


@pytest.mark.parametrize("h,w,pad", CE_F16)
def test_cross_entropy_dense_f16(L, h, w, pad):
    """fp16 storage (the reference instantiates the layer for half, cross_entropy.cpp:157-166):
    the fp32 oracle on the same binary16 inputs, 2e-3."""
    rng = np.random.default_rng(h * 11 + w)
    x = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float16).T)
    truth = np.asfortranarray((rng.uniform(-0.3, 1.0, (w, h)) * min(1.0, 4096.0 / h)).astype(np.float16).T)
    truth[0, :] = 0.0
    dy = rng.standard_normal(w).astype(np.float16)
    layer = L.cross_entropy_layer((h,))
    ld = h + pad
    half = torch.float16
    loss = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=half, ldim=ld),
                         L.DeviceMatrix.from_numpy(truth, dtype=half, ldim=ld))
    assert loss.dtype == half
    check(f"cross entropy f16 loss {h}x{w}", f32(loss.to_numpy()[0]), orc.cross_entropy_fwd(f32(x), f32(truth)), tol=TOL_F16)
    dym = L.DeviceMatrix.from_numpy(np.asfortranarray(dy.reshape(1, w)), dtype=half)
    dx, dt = layer.backward(dym)
    assert dx.dtype == half and dt.dtype == half
    rx, rt = orc.cross_entropy_bwd(f32(x), f32(truth), f32(dy))
    got = f32(dx.to_numpy())
    check(f"cross entropy f16 dx {h}x{w}", got, rx, tol=TOL_F16)
    assert np.all(got[f32(truth) <= 0] == 0.0)
    check(f"cross entropy f16 dtruth {h}x{w}", f32(dt.to_numpy()), rt, tol=TOL_F16)


@pytest.mark.parametrize("classes,spatial,w,pad", [(3, (8, 8), 23, 0), (10, (1,), 64, 0), (5, (7, 3), 9, 0),
                                                  (4, (6,), 5, 3), (21, (64, 64), 6, 0), (1000, (1,), 128, 0),
                                                  (2048, (1,), 16, 0), (1003, (1,), 70, 3), (37, (1,), 5000, 1)])
def test_cross_entropy_labels_f16(L, classes, spatial, w, pad):
    """Class indices stored as binary16 (exact up to 2048)."""
    rng = np.random.default_rng(classes * 101 + w)
    sp = int(np.prod(spatial))
    h = classes * sp
    x = np.asfortranarray(rng.uniform(0.05, 1.0, (w, h)).astype(np.float16).T)
    labels = np.asfortranarray(rng.integers(0, classes, (w, sp)).astype(np.float16).T)
    if sp > 2:
        labels[1, 0] = classes      # a label no class matches contributes nothing
        labels[2, 0] = -3.0
    elif w > 3:
        labels[0, 1] = classes
        labels[0, 2] = -3.0
    dy = rng.standard_normal(w).astype(np.float16)
    half = torch.float16
    layer = L.cross_entropy_layer((classes,) + tuple(spatial), use_labels=True)
    loss = layer.forward(L.DeviceMatrix.from_numpy(x, dtype=half, ldim=h + pad),
                         L.DeviceMatrix.from_numpy(labels, dtype=half, ldim=sp + pad)).to_numpy()
    check(f"cross entropy f16 (labels) loss {classes}x{sp}x{w}", f32(loss[0]),
          orc.cross_entropy_fwd(f32(x), f32(labels), True), tol=TOL_F16)
    dx, dt = layer.backward(L.DeviceMatrix.from_numpy(np.asfortranarray(dy.reshape(1, w)), dtype=half))
    assert dt is None
    rx, _ = orc.cross_entropy_bwd(f32(x), f32(labels), f32(dy), True)
    got = f32(dx.to_numpy())
    check(f"cross entropy f16 (labels) dx {classes}x{sp}x{w}", got, rx, tol=TOL_F16)
    assert np.array_equal(got == 0.0, rx == 0.0)


def test_cross_entropy_f16_rejects_mixed_types_and_odd_pointers(L):
    from lbann_amd import capi
    layer = L.cross_entropy_layer((8,))
    x = L.DeviceMatrix(8, 4, dtype=torch.float16, fill=0.5)
    t32 = L.DeviceMatrix(8, 4, fill=0.5)
    with pytest.raises(TypeError):
        layer.forward(x, t32)
    t = L.DeviceMatrix(8, 4, dtype=torch.float16, fill=0.5)
    loss = L.DeviceMatrix(1, 4, dtype=torch.float16)
    odd = capi.vp(x.tensor.data_ptr() + 1)
    rc = capi.lib().lbn_cross_entropy_fwd_f16(capi.vp(None), 4, 4, 0, 1, odd, 8, t.Buffer(), 8, loss.Buffer(), 1,
                                               capi.vp(None), 0)
    assert rc == -1
    # an empty mini-batch and an empty sample
    assert capi.lib().lbn_cross_entropy_fwd_f16(capi.vp(None), 8, 0, 0, 1, x.Buffer(), 8, t.Buffer(), 8,
                                                loss.Buffer(), 1, capi.vp(None), 0) == 0
    loss.tensor.fill_(7.0)
    assert capi.lib().lbn_cross_entropy_fwd_f16(capi.vp(None), 0, 4, 0, 1, capi.vp(None), 1, capi.vp(None), 1,
                                                loss.Buffer(), 1, capi.vp(None), 0) == 0
    torch.cuda.synchronize()
    assert (loss.to_numpy() == 0).all()


def test_cross_entropy_after_softmax(L):
    """softmax -> cross entropy and back, as in a classifier's last two layers."""
    rng = np.random.default_rng(3)
    h, w = 1000, 96
    logits = rand(rng, h, w, 0, 2)
    onehot = np.zeros((h, w), np.float32, order="F")
    onehot[rng.integers(0, h, w), np.arange(w)] = 1.0
    sm, ce = L.softmax_layer(), L.cross_entropy_layer((h,))
    p = sm.forward(L.DeviceMatrix.from_numpy(logits))
    loss = ce.forward(p, L.DeviceMatrix.from_numpy(onehot)).to_numpy()[0]
    dy = np.full(w, 1.0 / w, np.float32)
    dp, _ = ce.backward(vec_to_row(L, dy))
    dlogits = sm.backward(dp).to_numpy()
    p64 = orc.softmax_fwd(f64(logits))
    check("softmax+ce loss", loss, orc.cross_entropy_fwd(orc.softmax_fwd(logits), onehot), orc.cross_entropy_fwd(p64, f64(onehot)))
    # closed form of the composition: (softmax - onehot) / w
    assert rel_err(dlogits, (p64 - onehot) / w) < 5e-6


# ===================================================================== scale/bias layers
ESB_SHAPES = [
    # (h, w, ld_pad)   tile kernels with 64 and 256 rows per workgroup, column slabs, scalar fallback
    (105, 29, 0), (4096, 64, 0), (64, 1024, 0), (1024, 4096, 0), (256 * 512, 24, 0), (256 * 512 + 8, 5, 0),
    (2048, 17, 4), (1001, 7, 0), (130, 3, 3), (4, 300, 0), (1, 9, 0), (8192, 1, 0), (300000, 16, 0),
    (786432, 64, 0),   # a call that moves more than the last-level cache holds: streaming loads
]


@pytest.mark.parametrize("h,w,pad", ESB_SHAPES)
def test_entrywise_scale_bias(L, h, w, pad):
    rng = np.random.default_rng(h + 13 * w)
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    wts = np.asfortranarray(np.stack([rng.normal(1, 1, h), rng.normal(0, 1, h)], axis=1).astype(np.float32))
    layer = L.entrywise_scale_bias_layer((h,))
    layer.set_weights(wts[:, 0], wts[:, 1])
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    check(f"entrywise scale/bias y {h}x{w}", y, orc.entrywise_scale_bias_fwd(x, wts), orc.entrywise_scale_bias_fwd(f64(x), f64(wts)))
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    rdx, rwg = orc.entrywise_scale_bias_bwd(x, dy, wts)
    edx, ewg = orc.entrywise_scale_bias_bwd(f64(x), f64(dy), f64(wts))
    check(f"entrywise scale/bias dx {h}x{w}", dx, rdx, edx)
    check(f"entrywise scale/bias dweights {h}x{w}", layer.m_weights_gradient.to_numpy(), rwg, ewg)


CSB_CASES = [
    # dims (C, ...), w, ld_pad
    ((7, 5, 3), 23, 0), ((64, 56, 56), 8, 0), ((3, 224, 224), 4, 0), ((256, 4, 4), 32, 0), ((2048, 1, 1), 64, 0),
    ((5, 12), 10, 4), ((5, 13), 10, 0), ((1, 100000), 3, 0), ((2, 1), 1, 0), ((70000, 1), 2, 0), ((16, 128, 128), 16, 0),
    ((256, 28, 28), 24, 0), ((256, 7, 3), 200, 0),   # one 1024-thread workgroup per channel, vector and scalar
    ((8, 55, 55), 40, 0), ((4, 111, 111), 12, 0), ((2048, 7, 7), 16, 0),   # odd maps: row tiling with channel lookup
]


@pytest.mark.parametrize("dims,w,pad", CSB_CASES)
def test_channelwise_scale_bias(L, dims, w, pad):
    rng = np.random.default_rng(int(np.prod(dims)) + w)
    C, cs = dims[0], int(np.prod(dims[1:]))
    h = C * cs
    x, dy = rand(rng, h, w, 0.5, 2.0), rand(rng, h, w)
    wts = np.asfortranarray(np.stack([rng.normal(1, 1, C), rng.normal(0, 1, C)], axis=1).astype(np.float32))
    layer = L.channelwise_scale_bias_layer(dims)
    layer.set_weights(wts[:, 0], wts[:, 1])
    y = layer.forward(L.DeviceMatrix.from_numpy(x, ldim=h + pad)).to_numpy()
    check(f"channelwise scale/bias y {dims}x{w}", y, orc.channelwise_scale_bias_fwd(x, wts, C, cs),
          orc.channelwise_scale_bias_fwd(f64(x), f64(wts), C, cs))
    dx = layer.backward(L.DeviceMatrix.from_numpy(dy, ldim=h + pad)).to_numpy()
    rdx, rwg = orc.channelwise_scale_bias_bwd(x, dy, wts, C, cs)
    edx, ewg = orc.channelwise_scale_bias_bwd(f64(x), f64(dy), f64(wts), C, cs)
    check(f"channelwise scale/bias dx {dims}x{w}", dx, rdx, edx)
    check(f"channelwise scale/bias dweights {dims}x{w}", layer.m_weights_gradient.to_numpy(), rwg, ewg)


# ===================================================================== golden fixtures, boundary behaviour
def test_neighbour_layer_fixtures_on_gpu(L, golden):
    F32_EPS = np.finfo(np.float32).eps
    T = lambda a: np.asfortranarray(np.asarray(a).T)
    met = lambda y: float(np.mean(np.sum(np.asarray(y, np.float64) ** 2, axis=0)))
    pred = L.DeviceMatrix.from_numpy(T(golden["ce_prediction"]))
    loss = L.cross_entropy_layer((192,)).forward(pred, L.DeviceMatrix.from_numpy(T(golden["ce_dense_truth"]))).to_numpy()[0]
    assert rel_err(loss, golden["ce_loss_dense"]) < TOL_F32
    val = float(golden["ce_metric_dense"])
    assert abs(np.mean((1e-3 * loss.astype(np.float64)) ** 2) - val) <= val * float(golden["ce_metric_tol"])
    for dims in ((3, 8, 8), (3, 4, 4, 4)):   # the reference's 2-D and 3-D label cases
        loss = L.cross_entropy_layer(dims, use_labels=True).forward(
            pred, L.DeviceMatrix.from_numpy(T(golden["ce_labels"]))).to_numpy()[0]
        assert rel_err(loss, golden["ce_loss_labels"]) < TOL_F32
        val = float(golden["ce_metric_labels"])
        assert abs(np.mean((1e-3 * loss.astype(np.float64)) ** 2) - val) <= val * float(golden["ce_metric_tol"])
    esb = L.entrywise_scale_bias_layer((7, 5, 3))
    esb.set_weights(golden["esb_scale"], golden["esb_bias"])
    y = esb.forward(L.DeviceMatrix.from_numpy(T(golden["esb_x"]))).to_numpy()
    assert rel_err(y.T, golden["esb_y"]) < TOL_F32
    assert abs(met(y) - float(golden["esb_metric"])) <= 8 * float(golden["esb_metric"]) * F32_EPS
    csb = L.channelwise_scale_bias_layer((7, 5, 3))
    csb.set_weights(golden["csb_scale"], golden["csb_bias"])
    y = csb.forward(L.DeviceMatrix.from_numpy(T(golden["csb_x"]))).to_numpy()
    assert rel_err(y.T, golden["csb_y"]) < TOL_F32
    assert abs(met(y) - float(golden["csb_metric"])) <= 8 * float(golden["csb_metric"]) * F32_EPS


def test_neighbour_layers_empty_and_rejected_arguments(L):
    from lbann_amd import capi
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    null = capi.vp(None)
    lib = capi.lib()
    buf = torch.zeros(4096, device="cuda")
    p = capi.vp(buf.data_ptr())
    # empty inputs: nothing to do
    assert lib.lbn_entrywise_scale_bias_fwd_f32(st, 0, 4, null, 1, null, 1, null, 1) == 0
    assert lib.lbn_channelwise_scale_bias_fwd_f32(st, 4, 8, 0, null, 32, null, 32, null, 4) == 0
    assert lib.lbn_cross_entropy_fwd_f32(st, 8, 0, 0, 1, null, 8, null, 8, null, 1, null, 0) == 0
    assert lib.lbn_cross_entropy_bwd_f32(st, 0, 3, 0, 1, null, 1, null, 1, null, 1, null, 1, null, 1) == 0
    # a sample without entries has loss 0
    buf.fill_(7.0)
    assert lib.lbn_cross_entropy_fwd_f32(st, 0, 3, 0, 1, null, 1, null, 1, p, 1, null, 0) == 0
    torch.cuda.synchronize()
    assert buf[:3].tolist() == [0.0, 0.0, 0.0] and buf[3].item() == 7.0
    # rejected: leading dimension below the height, missing matrices, missing workspace
    assert lib.lbn_entrywise_scale_bias_fwd_f32(st, 8, 4, p, 4, p, 8, p, 8) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_entrywise_scale_bias_fwd_f32(st, 8, 4, p, 8, p, 8, p, 4) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_channelwise_scale_bias_bwd_f32(st, 2, 4, 4, p, 8, p, 8, null, 8, p, 2, p, 2, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_cross_entropy_fwd_f32(st, 8, 4, 1, 0, p, 8, p, 8, p, 1, null, 0) == capi.LBN_ERR_INVALID_ARGUMENT
    # dground_truth is optional (not written when NULL); given, its leading dimension must hold a column
    assert lib.lbn_cross_entropy_bwd_f32(st, 8, 4, 0, 1, p, 8, p, 8, p, 1, p, 8, null, 8) == 0
    assert lib.lbn_cross_entropy_bwd_f32(st, 8, 4, 0, 1, p, 8, p, 8, p, 1, p, 8, p, 4) == capi.LBN_ERR_INVALID_ARGUMENT
    big = torch.zeros(64 * 8192, device="cuda")
    pb = capi.vp(big.data_ptr())
    assert lib.lbn_entrywise_scale_bias_bwd_workspace_bytes(64, 8192) > 0
    assert lib.lbn_entrywise_scale_bias_bwd_f32(st, 64, 8192, pb, 64, pb, 64, pb, 64, p, 64, p, 64, null, 0) == capi.LBN_ERR_WORKSPACE
    assert lib.lbn_cross_entropy_fwd_f32(st, 65536, 8, 0, 1, pb, 65536, pb, 65536, p, 1, null, 0) == capi.LBN_ERR_WORKSPACE
    torch.cuda.synchronize()


# ===================================================================== gradient buffer
SINK_SHAPES = [
    # (h, w, contribution pad, gradient pad)
    (4096, 1, 0, 0), (8192, 2, 0, 0), (37, 5, 0, 0), (37, 5, 3, 1), (1, 1, 0, 0), (256, 2, 4, 8),
    (1026, 3, 2, 2), (3, 1000, 0, 1), (1 << 22, 1, 0, 0), ((1 << 21) + 1, 2, 0, 0), (2048, 2048, 0, 0),
]


@pytest.mark.parametrize("h,w,cpad,gpad", SINK_SHAPES)
def test_gradient_sink_bit_exact(L, h, w, cpad, gpad):
    """lbn_gradient_sink_f32 against the oracle's Scale + Axpy: same bits, padding untouched."""
    from lbann_amd import capi
    rng = np.random.default_rng(h + 31 * w)
    c = rand(rng, h, w)
    c[0, 0] = -0.0
    g0 = rand(rng, h, w)
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    dc = L.DeviceMatrix.from_numpy(c, ldim=h + cpad)
    for buf_scale, alpha in ((1.0, 1.0), (0.0, 1.0), (1.0, 0.37), (0.0, -2.5), (-1.25, 0.37)):
        dg = L.DeviceMatrix(h, w, ldim=h + gpad, fill=float("nan") if buf_scale == 0.0 else 123.0)
        if buf_scale != 0.0:
            dg.tensor[:, :h] = torch.from_numpy(np.ascontiguousarray(g0.T)).cuda()
        assert capi.lib().lbn_gradient_sink_f32(st, h, w, buf_scale, alpha, dc.Buffer(), dc.ldim, dg.Buffer(), dg.ldim) == 0
        got = dg.to_numpy()
        exp = orc.gradient_sink(g0, c, buf_scale, alpha)
        assert got.tobytes() == np.asfortranarray(exp).tobytes(), (buf_scale, alpha, rel_err(got, exp))
        if gpad:
            pad = dg.tensor[:, h:].cpu().numpy()
            assert (np.isnan(pad).all() if buf_scale == 0.0 else (pad == 123.0).all())


def test_gradient_buffer_takes_layer_norm_weight_gradients(L):
    """Two mini-batches through layer norm's backward, dscale / dbias handed to gradient
    buffers as the reference's bp_compute does (layer_norm.cpp:342-343): the first
    contribution overwrites an uninitialised buffer, the second accumulates."""
    rng = np.random.default_rng(342)
    n, w = 1024, 48
    gamma = rng.standard_normal(n).astype(np.float32)
    beta = rng.standard_normal(n).astype(np.float32)
    layer = L.layer_norm_layer((n,), scale=True, bias=True, scale_values=gamma, bias_values=beta)
    sink_s, sink_b = L.gradient_buffer(n), L.gradient_buffer(n)
    sink_s.gradient.tensor.fill_(float("nan"))
    sink_b.gradient.tensor.fill_(float("nan"))
    exp_s = exp_b = None
    for step in range(2):
        x, dy = rand(rng, n, w, 0.5, 2.0), rand(rng, n, w)
        layer.forward(L.DeviceMatrix.from_numpy(x))
        layer.backward(L.DeviceMatrix.from_numpy(dy))
        ds, db = layer.m_scale_gradient.to_numpy().reshape(n, 1), layer.m_bias_gradient.to_numpy().reshape(n, 1)
        sink_s.add_to_gradient(layer.m_scale_gradient, scale=1.0, sync_needed=True)
        sink_b.add_to_gradient(layer.m_bias_gradient, scale=1.0, sync_needed=True)
        exp_s = orc.gradient_sink(np.zeros((n, 1), np.float32) if step == 0 else exp_s, f32(ds), float(step), 1.0)
        exp_b = orc.gradient_sink(np.zeros((n, 1), np.float32) if step == 0 else exp_b, f32(db), float(step), 1.0)
        assert sink_s.status == sink_s.SYNC_NEEDED
    assert sink_s.gradient.to_numpy().tobytes() == exp_s.tobytes()
    assert sink_b.gradient.to_numpy().tobytes() == exp_b.tobytes()
    sink_s.finish_sync()
    sink_s.clear()
    assert sink_s.status == sink_s.CLEARED
    wrong = L.DeviceMatrix(n + 1, 1, fill=0.0)
    with pytest.raises(ValueError):
        sink_s.add_to_gradient(wrong)


def test_gradient_sink_empty_and_rejected_arguments(L):
    from lbann_amd import capi
    st = capi.vp(torch.cuda.current_stream().cuda_stream)
    null = capi.vp(None)
    lib = capi.lib()
    buf = torch.zeros(4096, device="cuda")
    p = capi.vp(buf.data_ptr())
    assert lib.lbn_gradient_sink_f32(st, 0, 4, 1.0, 1.0, null, 1, null, 1) == 0
    assert lib.lbn_gradient_sink_f32(st, 4, 0, 1.0, 1.0, null, 4, null, 4) == 0
    assert lib.lbn_gradient_sink_f32(st, -1, 4, 1.0, 1.0, p, 4, p, 4) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_gradient_sink_f32(st, 8, 4, 1.0, 1.0, p, 4, p, 8) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_gradient_sink_f32(st, 8, 4, 1.0, 1.0, p, 8, p, 4) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_gradient_sink_f32(st, 8, 4, 1.0, 1.0, null, 8, p, 8) == capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_gradient_sink_f32(st, 8, 4, 1.0, 1.0, p, 8, null, 8) == capi.LBN_ERR_INVALID_ARGUMENT
    torch.cuda.synchronize()
    assert float(buf.abs().sum()) == 0.0
