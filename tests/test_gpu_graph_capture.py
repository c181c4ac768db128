"""The entry points only enqueue work on the caller's stream (no synchronisation, no
allocation, no host read-back), so a caller may record them into a HIP graph.

Each case records one layer's fp_compute() + bp_compute() once and replays the graph
several times on new input contents, with eager work and synchronisations between the
replays; every replay must agree with an eager run of a fresh layer on the same data.
Shapes include those whose path is a register-resident cluster kernel: its rendezvous
tag is a per-call kernel argument, which a replay would repeat, so a recorded call also
records a node that advances a counter in the workspace, and the tag takes that in.  A
replay that saw the previous replay's partial results as its own would show here as
statistics of the previous data.
"""
import numpy as np
import pytest
import torch

from tests.parity import TOL_F16, TOL_F32, check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    from lbann_amd import layers
    layers.capi.lib()
    assert torch.cuda.is_available()
    return layers


def _outputs(layer, names):
    out = {"y": layer.activations, "dx": layer.error_signals}
    for n in names:
        out[n] = getattr(layer, n)
    return {k: np.array(v.to_numpy(), copy=True) for k, v in out.items()}


CASES = [
    # name, factory, h, w, dtype, extra outputs, input mean/std
    ("softmax rows", lambda L: L.softmax_layer(), 4096, 64, torch.float32, ()),
    ("softmax clusters", lambda L: L.softmax_layer(), 100000, 130, torch.float32, ()),
    ("log-softmax clusters", lambda L: L.log_softmax_layer(), 262148, 48, torch.float32, ()),
    ("channelwise softmax", lambda L: L.channelwise_softmax_layer((16, 512)), 8192, 32, torch.float32, ()),
    ("layer norm affine", lambda L: L.layer_norm_layer((2048,), 1e-5, True, True), 2048, 512, torch.float32,
     ("m_statistics", "m_statistics_gradient", "m_scale_gradient", "m_bias_gradient")),
    ("layer norm f16", lambda L: L.layer_norm_layer((4096,), 1e-5, True, True), 4096, 256, torch.float16,
     ("m_statistics", "m_scale_gradient", "m_bias_gradient")),
    ("layer norm clusters", lambda L: L.layer_norm_layer((150528,), 1e-5, True, True), 150528, 40, torch.float32,
     ("m_statistics", "m_statistics_gradient", "m_scale_gradient", "m_bias_gradient")),
    ("instance norm", lambda L: L.instance_norm_layer((8, 32, 32)), 8192, 24, torch.float32, ()),
    ("instance norm streaming clusters", lambda L: L.instance_norm_layer((2, 2400000)), 4800000, 2, torch.float32, ()),
    ("entry-wise batch norm", lambda L: L.entrywise_batch_normalization_layer((4096,)), 4096, 48, torch.float32,
     ("m_batch_statistics", "m_batch_statistics_gradient")),
    ("batch norm clusters", lambda L: L.batch_normalization_layer((64, 56, 56)), 64 * 3136, 16, torch.float32,
     ("m_mean_and_var", "m_mean_and_var_gradient", "m_scale_gradient", "m_bias_gradient")),
    ("batch norm f16", lambda L: L.batch_normalization_layer((32, 28, 28)), 32 * 784, 16, torch.float16,
     ("m_mean_and_var", "m_scale_gradient", "m_bias_gradient")),
    ("entry-wise scale/bias", lambda L: L.entrywise_scale_bias_layer((512,)), 512, 2048, torch.float32,
     ("m_weights_gradient",)),
    ("channel-wise scale/bias", lambda L: L.channelwise_scale_bias_layer((8, 64, 64)), 8 * 4096, 16, torch.float32,
     ("m_weights_gradient",)),
    ("batch norm clusters in turn", lambda L: L.batch_normalization_layer((1500, 4, 4)), 1500 * 16, 600, torch.float32,
     ("m_mean_and_var", "m_mean_and_var_gradient", "m_scale_gradient", "m_bias_gradient")),
    ("batch norm streaming clusters", lambda L: L.batch_normalization_layer((3, 1200000)), 3600000, 2, torch.float32,
     ("m_mean_and_var", "m_mean_and_var_gradient", "m_scale_gradient", "m_bias_gradient")),
    ("batch norm small", lambda L: L.batch_normalization_layer((7, 5, 3)), 105, 14, torch.float32,
     ("m_mean_and_var", "m_mean_and_var_gradient")),
]


@pytest.mark.parametrize("name,make,h,w,dtype,extra", CASES, ids=[c[0] for c in CASES])
def test_graph_replay_matches_eager(L, name, make, h, w, dtype, extra):
    gen = torch.Generator(device="cuda").manual_seed(h * 31 + w)
    tol = TOL_F16 if dtype == torch.float16 else TOL_F32

    def new_data(k):
        x = (torch.randn((w, h), generator=gen, device="cuda") * (1.0 + k) + 0.5 * k).to(dtype)
        dy = torch.randn((w, h), generator=gen, device="cuda").to(dtype)
        return x, dy

    x, dy = L.DeviceMatrix(h, w, dtype=dtype), L.DeviceMatrix(h, w, dtype=dtype)
    x0, dy0 = new_data(0)
    x.tensor.copy_(x0), dy.tensor.copy_(dy0)
    layer = make(L)
    layer.forward(x), layer.backward(dy)  # eager first: sizes outputs and scratch
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.fp_compute()
        layer.bp_compute()

    for k in range(1, 6):
        xk, dyk = new_data(k)
        x.tensor.copy_(xk), dy.tensor.copy_(dyk)
        graph.replay()
        torch.cuda.synchronize()
        got = _outputs(layer, extra)

        fresh = make(L)  # eager run on the same data (running statistics differ and are left out)
        fx, fdy = L.DeviceMatrix(h, w, dtype=dtype), L.DeviceMatrix(h, w, dtype=dtype)
        fx.tensor.copy_(xk), fdy.tensor.copy_(dyk)
        fresh.forward(fx), fresh.backward(fdy)
        torch.cuda.synchronize()
        want = _outputs(fresh, extra)
        for key in got:
            check(f"{name} replay {k}: {key}", got[key], want[key], tol=2 * tol)
