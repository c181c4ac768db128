"""The bounded wait of the kernels in which workgroups wait for each other: its designed
give-up exit, driven from the host (one workgroup polls for a partner that is never launched,
with a budget of a few polls), and how both host-side mirrors report it.  Every kernel here
exits normally."""
import ctypes

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


def _flag(L, ws):
    flag = L.capi.cint(0)
    L.call("lbn_workspace_timed_out", L._stream(), L.capi.vp(ws.data_ptr()), flag)
    return flag.value


def test_wait_gives_up_sets_the_flag_and_the_kernel_ends(L):
    lib = L.capi.lib()
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    out = torch.full((4,), float("nan"), device="cuda")
    assert _flag(L, ws) == 0
    status = lib.lbn_selftest_cluster_wait_gives_up(L._stream(), L.capi.vp(ws.data_ptr()), 4096, 64,
                                                    L.capi.vp(out.data_ptr()))
    assert status == 0
    torch.cuda.synchronize()                       # returns: the wave left its loop and the kernel ended
    assert _flag(L, ws) == 1                        # ... and said so
    assert out.cpu().tolist() == [1.0, 2.0, -1.0, -1.0]   # member 0's own pair; stand-ins for the absent member
    assert _flag(L, ws) == 1                        # sticky until the header is cleared
    ws[:64].zero_()
    assert _flag(L, ws) == 0
    # rejected arguments launch nothing
    assert lib.lbn_selftest_cluster_wait_gives_up(L._stream(), L.capi.vp(ws.data_ptr()), 4096, 64, None) == L.capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_selftest_cluster_wait_gives_up(L._stream(), L.capi.vp(ws.data_ptr()), 4096, 0, L.capi.vp(out.data_ptr())) == L.capi.LBN_ERR_INVALID_ARGUMENT
    assert lib.lbn_selftest_cluster_wait_gives_up(L._stream(), L.capi.vp(ws.data_ptr()), 64, 64, L.capi.vp(out.data_ptr())) == L.capi.LBN_ERR_WORKSPACE


def test_python_mirror_reports_a_wait_that_gave_up(L):
    rng = np.random.default_rng(11)
    x = np.asfortranarray(rng.standard_normal((4, 100000), dtype=np.float32).T)   # uses scratch
    layer = L.softmax_layer()
    y = layer.forward(L.DeviceMatrix.from_numpy(x))
    check("softmax before", y.to_numpy(), orc.softmax_fwd(x), orc.softmax_fwd(np.asfortranarray(x.astype(np.float64))))
    ws = layer._ws.buf
    assert ws is not None and ws.numel() >= 128 and _flag(L, ws) == 0
    out = torch.empty(4, device="cuda")
    L.call("lbn_selftest_cluster_wait_gives_up", L._stream(), L.capi.vp(ws.data_ptr()), ws.numel(), 16,
           L.capi.vp(out.data_ptr()))
    with pytest.raises(L.ClusterWaitTimedOut):
        y = layer.forward(L.DeviceMatrix.from_numpy(x))  # the next call registers the workspace for checking
        y.to_numpy()                                     # results are consumed here: the raised word surfaces
        # (with LBN_CHECK_CLUSTER_WAITS=1 in the environment the call itself raises)
    assert _flag(L, ws) == 0                             # reported once, then cleared
    y = layer.forward(L.DeviceMatrix.from_numpy(x))
    check("softmax after", y.to_numpy(), orc.softmax_fwd(x), orc.softmax_fwd(np.asfortranarray(x.astype(np.float64))))


def test_cpp_adapter_reports_a_wait_that_gave_up(L):
    from tests.test_cpp_adapter import driver, vp
    d = driver()
    rng = np.random.default_rng(12)
    h, w = 100000, 4
    x = np.asfortranarray(rng.standard_normal((w, h), dtype=np.float32).T)
    mx, my = L.DeviceMatrix.from_numpy(x), L.DeviceMatrix(h, w, fill=float("nan"))
    out = torch.empty(4, device="cuda")
    err = ctypes.create_string_buffer(512)
    rc = d.drv_cluster_wait_check(ctypes.c_int64(h), ctypes.c_int64(w), mx.Buffer(), my.Buffer(), vp(out.data_ptr()),
                                  vp(torch.cuda.current_stream().cuda_stream), err, 512)
    assert rc == 0, err.value.decode()
    assert b"ran out" in err.value                       # the message of the exception that was thrown and caught
    check("adapter softmax after", my.to_numpy(), orc.softmax_fwd(x), orc.softmax_fwd(np.asfortranarray(x.astype(np.float64))))
