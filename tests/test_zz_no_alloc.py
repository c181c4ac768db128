"""The softmax forward entry point that allocates nothing (its scratch is an array inside
the library's code object) against lbn_softmax_fwd_f32 with a caller-provided workspace:
the same kernels on the same inputs, so the outputs must agree bit for bit.  Two calls in
a row on one GPU share the array, the second with a smaller input; both shapes take the
paths that use scratch (partial sums of the split kernels, cluster slots)."""
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


def _pair(L, x):
    """(output of the static-scratch entry point, output of the workspace entry point)."""
    lib = L.capi.lib()
    h, w = x.shape
    xd = L.DeviceMatrix.from_numpy(x)
    y_static = L.DeviceMatrix(h, w, fill=float("nan"))
    y_ws = L.DeviceMatrix(h, w, fill=float("nan"))
    nbytes = lib.lbn_softmax_workspace_bytes(h, w)
    assert 0 < nbytes <= lib.lbn_softmax_fwd_static_scratch_max_bytes(), "shape must use scratch and fit"
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    st = L._stream()
    L.call("lbn_softmax_fwd_static_scratch_f32", st, h, w, xd.Buffer(), xd.ldim, y_static.Buffer(), y_static.ldim)
    L.call("lbn_softmax_fwd_f32", st, h, w, xd.Buffer(), xd.ldim, y_ws.Buffer(), y_ws.ldim,
           L.capi.vp(ws.data_ptr()), nbytes)
    torch.cuda.synchronize()
    return y_static.to_numpy(), y_ws.to_numpy()


def test_static_scratch_softmax_two_calls_in_a_row(L):
    rng = np.random.default_rng(0x4C42000B)
    # first call: rows of 262144 entries, 64 MiB per tensor (several workgroups share a row and
    # meet through the scratch); second call, smaller: 100000 x 8 (split kernels, partial sums)
    for h, w in ((262144, 64), (100000, 8)):
        x = np.asfortranarray((2.0 * rng.standard_normal((w, h), dtype=np.float32)).T)
        got, ref = _pair(L, x)
        assert got.tobytes() == ref.tobytes(), f"{h}x{w}: static-scratch output differs from the workspace entry point"
        assert np.abs(got.astype(np.float64).sum(axis=0) - 1.0).max() < 1e-4
        if h * w <= 1 << 20:
            # 100000 sequential fp32 additions per column: the float64 leg of the gate applies
            check(f"static scratch softmax {h}x{w}", got, orc.softmax_fwd(x),
                  orc.softmax_fwd(np.asfortranarray(x.astype(np.float64))))


def test_static_scratch_softmax_rejects_what_does_not_fit(L):
    lib = L.capi.lib()
    # 4096 columns of 40000 entries would need 4 MiB of slots: rejected before any launch,
    # so the (too small) buffers passed here are never touched
    h, w = 40000, 4096
    assert lib.lbn_softmax_workspace_bytes(h, w) > lib.lbn_softmax_fwd_static_scratch_max_bytes()
    small = L.DeviceMatrix(16, 1)
    status = lib.lbn_softmax_fwd_static_scratch_f32(L._stream(), h, w, small.Buffer(), h, small.Buffer(), h)
    assert status == L.capi.LBN_ERR_UNSUPPORTED
    assert lib.lbn_softmax_fwd_static_scratch_f32(L._stream(), 0, 0, None, 0, None, 0) == 0
    # shapes that need no scratch at all go straight through
    x = np.asfortranarray(np.random.default_rng(5).standard_normal((7, 1024), dtype=np.float32).T)
    xd, yd = L.DeviceMatrix.from_numpy(x), L.DeviceMatrix(1024, 7)
    L.call("lbn_softmax_fwd_static_scratch_f32", L._stream(), 1024, 7, xd.Buffer(), xd.ldim, yd.Buffer(), yd.ldim)
    check("static scratch softmax 1024x7", yd.to_numpy(), orc.softmax_fwd(x))


def _static_flag(L):
    flag = ctypes.c_int(-1)
    L.call("lbn_softmax_fwd_static_scratch_timed_out", L._stream(), flag)
    return flag.value


def test_static_scratch_wait_that_gives_up_is_seen_and_cleared(L):
    """The bounded waits' sticky word lives in the library-owned array on this path: the
    host-driven give-up (one member of a cluster of two, a budget of a few polls; the kernel
    exits normally) raises it there, the dedicated call reads and clears it, and the entry
    point works as before afterwards."""
    lib = L.capi.lib()
    assert lib.lbn_softmax_fwd_static_scratch_prepare() == 0
    assert lib.lbn_softmax_fwd_static_scratch_prepare() == 0     # again: harmless
    assert _static_flag(L) == 0
    out = torch.full((4,), float("nan"), device="cuda")
    # NULL workspace = the library's own array
    L.call("lbn_selftest_cluster_wait_gives_up", L._stream(), None, 0, 32, L.capi.vp(out.data_ptr()))
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [1.0, 2.0, -1.0, -1.0]
    assert _static_flag(L) == 1      # seen ...
    assert _static_flag(L) == 0      # ... and cleared by that read
    assert lib.lbn_softmax_fwd_static_scratch_timed_out(L._stream(), None) == L.capi.LBN_ERR_INVALID_ARGUMENT
    rng = np.random.default_rng(0x4C42000C)
    x = np.asfortranarray((2.0 * rng.standard_normal((8, 100000), dtype=np.float32)).T)
    got, ref = _pair(L, x)
    assert got.tobytes() == ref.tobytes()
    assert _static_flag(L) == 0
