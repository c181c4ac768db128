"""The five layers for TensorDataType = double (lbn_*_f64) against the float64 evaluation of the
restated reference code.  Tolerance 1e-10: both sides compute in binary64, the reference with
sequential sums (n * 1e-16 of rounding), the GPU with trees."""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import TOL_F64, check

pytestmark = pytest.mark.gpu
F64 = torch.float64


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()
    assert torch.cuda.is_available()
    return layers


def rand(rng, h, w, mean=0.0, std=1.0):
    return np.asfortranarray((rng.standard_normal((w, h)) * std + mean).T)


def up(L, a, pad=0):
    return L.DeviceMatrix.from_numpy(a, dtype=F64, ldim=a.shape[0] + pad if pad else None)


# (height, width, padding of the leading dimension)
SM_CASES = [(1, 5, 0), (2, 3, 0), (7, 9, 0), (64, 33, 0), (100, 17, 2), (1001, 40, 0), (1001, 40, 1), (4096, 64, 0),
            (32768, 40, 0), (30522, 24, 0), (50257, 6, 1), (70000, 5, 0), (262144, 3, 0), (16, 4096, 0),
            (128, 2048, 0), (10, 20000, 0),
            # backward with dy partly in LDS (16386 to 32768 entries), more rows than compute units
            (20000, 300, 2), (32766, 520, 0), (16386, 257, 0)]


@pytest.mark.parametrize("kind", ["softmax", "log_softmax"])
@pytest.mark.parametrize("h,w,pad", SM_CASES)
def test_softmax_family_f64(L, kind, h, w, pad):
    rng = np.random.default_rng(h * 131 + w)
    x, dy = rand(rng, h, w, 0.0, 2.0), rand(rng, h, w)
    if h > 100:
        x[rng.integers(0, h, size=max(1, h // 100)), :] = 30.0   # max-subtraction matters
    layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
    fwd, bwd = ((orc.softmax_fwd, orc.softmax_bwd) if kind == "softmax" else (orc.log_softmax_fwd, orc.log_softmax_bwd))
    y = layer.forward(up(L, x, pad)).to_numpy()
    assert y.dtype == np.float64
    check(f"f64 {kind} y {h}x{w}", y, fwd(x), tol=TOL_F64)
    # backward on outputs without a dominant entry: with y_k = 1 - 1e-11 the expression
    # y_k (dy_k - sum) cancels to 1e-11 of its terms in any summation order, binary64 included
    y = layer.forward(up(L, rand(rng, h, w, 0.0, 2.0), pad)).to_numpy()
    dx = layer.backward(up(L, dy, pad)).to_numpy()
    check(f"f64 {kind} dx {h}x{w}", dx, bwd(y, dy), tol=TOL_F64)


def test_softmax_f64_in_place_and_special_values(L):
    rng = np.random.default_rng(5)
    x = rand(rng, 515, 12, 0.0, 3.0)
    x[3, 0] = -np.inf
    x[:, 1] = -1e300           # every exponential is exp(0)
    x[:, 2] = np.linspace(-745, 0, 515)   # results reach the denormal range: flushed to 0 by softmax
    x[5, 3] = np.nan
    xm = up(L, x)
    layer = L.softmax_layer()
    y = layer.forward(xm, in_place=True).to_numpy()
    check("f64 softmax special y", y, orc.softmax_fwd(x), tol=TOL_F64)
    # non-normal results (denormals, and the NaNs of the column that holds one) are flushed to 0
    assert (y[:, 2] == 0).sum() > 0 and (y[:, 3] == 0).all()
    dy = rand(rng, 515, 12)
    dx = layer.backward(up(L, dy), in_place=True).to_numpy()
    check("f64 softmax special dx", dx, orc.softmax_bwd(y, dy), tol=TOL_F64)


def test_softmax_f64_long_rows_in_place(L):
    """Rows of 24000 doubles, more rows than compute units: the backward kernel that walks rows with
    dy partly in LDS writes dx over dy."""
    rng = np.random.default_rng(77)
    h, w = 24000, 300
    x, dy = rand(rng, h, w, 0.0, 2.0), rand(rng, h, w)
    for kind, fwd, bwd in (("softmax", orc.softmax_fwd, orc.softmax_bwd),
                           ("log_softmax", orc.log_softmax_fwd, orc.log_softmax_bwd)):
        layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
        y = layer.forward(up(L, x)).to_numpy()
        dx = layer.backward(up(L, dy), in_place=True).to_numpy()
        check(f"f64 {kind} dx in place {h}x{w}", dx, bwd(y, dy), tol=TOL_F64)


@pytest.mark.parametrize("dims,dim,single,w,pad", [((8, 256), 0, False, 24, 0), ((5, 7, 3), 0, False, 9, 0),
                                                  ((64, 4096), 0, False, 4, 0), ((3, 40001), 0, False, 5, 1),
                                                  ((12, 16, 10), -1, True, 6, 0), ((6, 50), -1, True, 33, 0),
                                                  # channels of 16386 to 32768 entries: backward with dy partly in LDS
                                                  ((3, 20000), 0, False, 100, 0), ((2, 32768), 0, False, 3, 2)])
def test_channelwise_softmax_f64(L, dims, dim, single, w, pad):
    h = int(np.prod(dims))
    rng = np.random.default_rng(h + w)
    x, dy = rand(rng, h, w), rand(rng, h, w)
    layer = L.channelwise_softmax_layer(dims, dim, single)
    cs, stride, C = layer.get_channel_size_and_stride()
    y = layer.forward(up(L, x, pad)).to_numpy()
    check(f"f64 channelwise y {dims}", y, orc.channelwise_softmax_fwd(x, C, cs, stride), tol=TOL_F64)
    dx = layer.backward(up(L, dy, pad)).to_numpy()
    check(f"f64 channelwise dx {dims}", dx, orc.channelwise_softmax_bwd(y, dy, C, cs, stride), tol=TOL_F64)


LN_CASES = [((1024,), 0, 128, True, 0), ((31,), 0, 15, True, 0), ((8, 512), -1, 9, True, 0), ((1,), 0, 6, True, 0),
            ((3, 777), 1, 11, True, 1), ((4096,), 0, 300, True, 0), ((4096,), 0, 2100, True, 0), ((64,), 0, 5000, False, 0),
            ((40000,), 0, 4, True, 0), ((70001,), 0, 3, True, 0), ((2, 20000), 1, 3, False, 2), ((16384,), 0, 20, True, 0),
            ((128,), 0, 9000, True, 0)]


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dims,start_dim,w,affine,pad", LN_CASES)
def test_layer_norm_f64(L, dims, start_dim, w, affine, pad, mode):
    h = int(np.prod(dims))
    rng = np.random.default_rng(h * 7 + w)
    x, dy = rand(rng, h, w, 0.3, 1.5), rand(rng, h, w)
    n = int(np.prod(dims[(start_dim if start_dim >= 0 else len(dims) + start_dim):]))
    scale, bias = 1 + 0.3 * rng.standard_normal(n), 0.3 * rng.standard_normal(n)
    kw = dict(scale_values=scale, bias_values=bias) if affine else {}
    layer = L.layer_norm_layer(dims, 1e-5, affine, affine, start_dim, datatype=F64,
                               stats_mode=L.LBN_STATS_SUMSQ if mode else L.LBN_STATS_TWO_PASS, **kw)
    G = layer.num_normalized
    y = layer.forward(up(L, x, pad)).to_numpy()
    stats = layer.m_statistics.to_numpy()
    sc, bi = (scale, bias) if affine else (None, None)
    y_ref, st_ref = orc.layer_norm_fwd(x, G, n, n, 1e-5, sc, bi)
    check(f"f64 layer_norm stats {dims} w={w}", stats, st_ref, tol=TOL_F64)
    check(f"f64 layer_norm y {dims} w={w}", y, y_ref, tol=TOL_F64)
    dx = layer.backward(up(L, dy, pad)).to_numpy()
    dx_ref, sg_ref, dg_ref, db_ref = orc.layer_norm_bwd(x, dy, st_ref, G, n, n, 1e-5, sc, affine, affine)
    check(f"f64 layer_norm dx {dims} w={w}", dx, dx_ref, tol=TOL_F64)
    if n > 1:
        check(f"f64 layer_norm stats grad {dims} w={w}", layer.m_statistics_gradient.to_numpy(), sg_ref, tol=TOL_F64)
    if affine:
        check(f"f64 layer_norm dscale {dims} w={w}", layer.m_scale_gradient.to_numpy(), dg_ref, tol=TOL_F64)
        check(f"f64 layer_norm dbias {dims} w={w}", layer.m_bias_gradient.to_numpy(), db_ref, tol=TOL_F64)


BN_CASES = [((8, 16, 16), 12, True, 0, True), ((7, 5, 3), 14, False, 0, True), ((5, 24), 10, True, 8, True),
            ((3, 1001), 7, True, 3, True), ((4, 1), 1, True, 0, True), ((6, 1), 33, True, 0, True),
            ((64, 28, 28), 16, True, 0, True), ((3, 56, 56), 16, True, 0, False), ((256, 14, 14), 32, False, 0, True),
            ((2, 100000), 3, True, 0, True), ((1024, 2, 2), 64, True, 0, True),
            # channels of 128 KB to 400 KB, at least one per compute unit: one workgroup keeps a channel
            ((256, 28, 28), 64, True, 0, True), ((300, 14, 14), 100, False, 2, True), ((257, 10, 10), 201, True, 0, True),
            ((600, 6, 14), 196, True, 0, True)]


@pytest.mark.parametrize("dims,w,bessel,pad,training", BN_CASES)
def test_batch_norm_f64(L, dims, w, bessel, pad, training):
    h = int(np.prod(dims))
    rng = np.random.default_rng(h * 13 + w)
    x, dy = rand(rng, h, w, 2.0, 3.0), rand(rng, h, w)
    C = dims[0]
    cs = h // C
    scale, bias = rng.uniform(0.5, 1.5, C), 0.1 * rng.standard_normal(C)
    layer = L.batch_normalization_layer(dims, 0.9, 1e-5, bessel, scale, bias, datatype=F64)
    layer.training = training
    rm0, rv0 = 0.1 * np.arange(C, dtype=np.float64), 1.0 + 0.05 * np.arange(C, dtype=np.float64)
    layer.weights[2].tensor[:C] = torch.from_numpy(rm0).cuda()
    layer.weights[3].tensor[:C] = torch.from_numpy(rv0).cuda()
    y = layer.forward(up(L, x, pad)).to_numpy()
    mv = layer.m_mean_and_var.to_numpy()
    dx = layer.backward(up(L, dy, pad)).to_numpy()
    mvg = layer.m_mean_and_var_gradient.to_numpy()
    rm, rv = rm0.copy(), rv0.copy()
    y_ref, m_ref, v_ref = orc.batch_norm_fwd(x, C, cs, 1e-5, 0.9, scale, bias, rm, rv, bessel, training)
    dx_ref, dg_ref, db_ref, dm_ref, dv_ref = orc.batch_norm_bwd(x, dy, C, cs, 1e-5, m_ref, v_ref, scale, rm, rv, bessel,
                                                                training)
    tag = f"dims={dims} w={w}"
    check(f"f64 batch_norm y {tag}", y, y_ref, tol=TOL_F64)
    if training:
        check(f"f64 batch_norm mean {tag}", mv[:, 0], m_ref, tol=TOL_F64)
        check(f"f64 batch_norm var {tag}", mv[:, 1], v_ref, tol=TOL_F64)
    check(f"f64 batch_norm rmean {tag}", layer.weights[2].to_numpy(), rm, tol=TOL_F64)
    check(f"f64 batch_norm rvar {tag}", layer.weights[3].to_numpy(), rv, tol=TOL_F64)
    check(f"f64 batch_norm dx {tag}", dx, dx_ref, tol=TOL_F64)
    check(f"f64 batch_norm dscale {tag}", layer.m_scale_gradient.to_numpy(), dg_ref, tol=TOL_F64)
    check(f"f64 batch_norm dbias {tag}", layer.m_bias_gradient.to_numpy(), db_ref, tol=TOL_F64)
    check(f"f64 batch_norm dmean {tag}", mvg[:, 0], dm_ref, tol=TOL_F64)
    check(f"f64 batch_norm dvar {tag}", mvg[:, 1], dv_ref, tol=TOL_F64)


def test_f64_rejected_arguments(L):
    lib = L.capi.lib()
    st = L._stream()
    small = L.DeviceMatrix(16, 1, dtype=F64)
    p = small.Buffer()
    assert lib.lbn_softmax_fwd_f64(st, -1, 4, p, 16, p, 16) == L.capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_softmax_fwd_f64(st, 16, 2, p, 8, p, 16) == L.capi.LBN_ERR_INVALID_ARGUMENT   # ld < height
    assert lib.lbn_softmax_fwd_f64(st, 0, 0, None, 0, None, 0) == 0
    assert lib.lbn_layer_norm_bwd_f64(st, 1, 16, 16, 1, 1e-5, p, 16, p, 16, p, 16, p, 2, p, 2, None, p, None, None,
                                      0) == L.capi.LBN_ERR_INVALID_ARGUMENT                  # dscale without scale
    assert lib.lbn_layer_norm_bwd_f64(st, 1, 16, 16, 1, 1e-5, p, 16, p, 16, p, 16, p, 2, p, 2, p, p, None, None,
                                      0) == L.capi.LBN_ERR_WORKSPACE
    assert lib.lbn_batch_norm_fwd_f64(st, 2, 8, 1, 1, 1e-5, 0.9, 1, p, 16, p, 16, p, p, p, p, p, p, None, 0,
                                      0) == L.capi.LBN_ERR_WORKSPACE
