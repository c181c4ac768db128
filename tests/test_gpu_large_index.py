"""Matrices with more than 2^31 entries (8.8 GB per fp32 tensor): element offsets no longer
fit 32 bits, so every kernel's addressing is exercised beyond that limit.  The full tensors
are checked through size-independent properties computed on the GPU (softmax columns sum
to 1, normalised rows have mean 0 and variance 1, gradients sum to 0, ...), and a handful of
columns, the last one included, are compared with the CPU oracle.
"""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as orc
from tests.parity import TOL_F32, check

pytestmark = pytest.mark.gpu

H, W = 4096, 540000          # 2 211 840 000 entries
assert H * W > 2 ** 31


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()
    assert torch.cuda.is_available()
    if torch.cuda.get_device_properties(0).total_memory < 100 * 2 ** 30:
        pytest.skip("needs 100 GiB of device memory")
    return layers


def _fill(m, mean, std, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    # normal_ in slabs: one call over 2^31+ entries is not needed and slabs keep the generator cheap
    for c0 in range(0, m.width, 60000):
        m.tensor[c0:c0 + 60000].normal_(mean, std, generator=gen)
    return m


def _cols(m, cols):
    """(height x len(cols)) column-major host copy of the chosen columns."""
    return np.asfortranarray(m.tensor[cols, : m.height].float().cpu().numpy().T)


COLS = [0, 1, 262143, 524288, W - 2, W - 1]   # the last ones lie beyond element 2^31


def test_softmax_beyond_2g_entries(L):
    x = _fill(L.DeviceMatrix(H, W), 0.0, 2.0, 1)
    layer = L.softmax_layer()
    y = layer.forward(x)
    assert torch.allclose(y.tensor.sum(dim=1), torch.ones(W, device="cuda"), atol=2e-5)
    xc, yc = _cols(x, COLS), _cols(y, COLS)
    check("softmax y (columns of a 2.2G-entry matrix)", yc, orc.softmax_fwd(xc))
    dy = x                       # reuse the input buffer as dL/dy: any values do
    dx = layer.backward(dy)
    assert float(dx.tensor.sum(dim=1).abs().max()) < 1e-4
    check("softmax dx", _cols(dx, COLS), orc.softmax_bwd(yc, xc))


def test_layer_norm_beyond_2g_entries(L):
    x = _fill(L.DeviceMatrix(H, W), 0.5, 1.5, 2)
    scale = np.linspace(0.5, 1.5, H).astype(np.float32)
    bias = np.linspace(-0.2, 0.2, H).astype(np.float32)
    layer = L.layer_norm_layer((H,), 1e-5, True, True, 0, scale, bias)
    y = layer.forward(x)
    xc = _cols(x, COLS)
    y_ref, st_ref = orc.layer_norm_fwd(xc, 1, H, H, 1e-5, scale, bias)
    check("layer norm y", _cols(y, COLS), y_ref)
    check("layer norm stats", _cols(layer.m_statistics, COLS), st_ref)
    # every row: mean of x matches the stored statistic
    assert torch.allclose(layer.m_statistics.tensor[:, 0], x.tensor.mean(dim=1), atol=1e-4)
    dy = y                       # reuse the output buffer as dL/dy
    dyc = _cols(dy, COLS)
    dx = layer.backward(dy)
    dx_ref, sg_ref, _, _ = orc.layer_norm_bwd(xc, dyc, st_ref, 1, H, H, 1e-5, scale, True, True)
    check("layer norm dx", _cols(dx, COLS), dx_ref)
    check("layer norm stats grad", _cols(layer.m_statistics_gradient, COLS), sg_ref)
    # dbias is the sum of dy over all rows: torch's reduction over the 2.2G entries as the yardstick
    db = layer.m_bias_gradient.tensor[:H]
    ref = dy.tensor[:, :H].double().sum(dim=0)
    assert float(((db.double() - ref).abs() / (ref.abs() + 1.0)).max()) < 1e-3


def test_batch_norm_beyond_2g_entries(L):
    C, cs = 8, 512
    x = _fill(L.DeviceMatrix(C * cs, W), 2.0, 3.0, 3)       # h = 4096: 8 channels of 512 entries
    layer = L.batch_normalization_layer((C, cs))
    y = layer.forward(x)
    mv = layer.m_mean_and_var.to_numpy()
    xs = x.tensor[:, : C * cs].reshape(W, C, cs)
    mean_ref = xs.double().mean(dim=(0, 2)).cpu().numpy()
    var_ref = xs.double().var(dim=(0, 2), unbiased=True).cpu().numpy()
    assert np.allclose(mv[:, 0], mean_ref, rtol=1e-5, atol=1e-5) and np.allclose(mv[:, 1], var_ref, rtol=1e-4)
    ys = y.tensor[:, : C * cs].reshape(W, C, cs)
    assert float(ys.double().mean(dim=(0, 2)).abs().max()) < 1e-4
    assert float((ys.double().var(dim=(0, 2), unbiased=True) - 1.0).abs().max()) < 1e-3
    # the last column against the closed form with the kernel's own statistics
    last = _cols(x, [W - 1])[:, 0].reshape(C, cs)
    want = (last - mv[:, :1]) / np.sqrt(mv[:, 1:] + 1e-5)
    check("batch norm y, last column", _cols(y, [W - 1])[:, 0].reshape(C, cs), want.astype(np.float32))
    dy = y
    dx = layer.backward(dy)
    ds = dx.tensor[:, : C * cs].reshape(W, C, cs)
    assert float(ds.double().mean(dim=(0, 2)).abs().max()) < 1e-5     # dx sums to zero over a channel


def test_entrywise_layers_beyond_2g_entries(L):
    x = _fill(L.DeviceMatrix(H * 128, W // 128 + 1), 0.5, 2.0, 4)     # 524288 x 4219: tall
    h, w = x.height, x.width
    assert h * w > 2 ** 31
    wts = np.stack([np.linspace(0.5, 1.5, h), np.linspace(-1, 1, h)], axis=1).astype(np.float32)
    layer = L.entrywise_scale_bias_layer((h,))
    layer.set_weights(wts[:, 0], wts[:, 1])
    y = layer.forward(x)
    cols = [0, w // 2, w - 1]
    xc = _cols(x, cols)
    check("entrywise scale/bias y", _cols(y, cols), orc.entrywise_scale_bias_fwd(xc, np.asfortranarray(wts)))
    dx = layer.backward(y)       # dy = y
    check("entrywise scale/bias dx", _cols(dx, cols), wts[:, :1] * _cols(y, cols))
    wg = layer.m_weights_gradient.to_numpy()
    rows = [0, 12345, h - 1]
    for r in rows:
        xr, yr = x.tensor[:, r].double(), y.tensor[:, r].double()
        assert abs(wg[r, 0] - float((xr * yr).sum())) <= 1e-4 * float((xr * yr).abs().sum())
        assert abs(wg[r, 1] - float(yr.sum())) <= 1e-4 * float(yr.abs().sum())
