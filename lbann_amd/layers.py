"""Host-side mirror of the LBANN layer classes (layer norm, batch norm, softmax, log-softmax,
channelwise softmax; instance norm, entry-wise batch norm, cross entropy and the two scale/bias
layers), over the C ABI.

Each class keeps the reference layer's constructor parameters, its member
matrices and its two compute hooks, `fp_compute()` and `bp_compute()`
(include/lbann/layers/layer.hpp:835,852), and forwards them to liblbnorm.so.
A harness plays the role of data_type_layer::forward_prop / back_prop_impl_
(src/layers/data_type_layer.cpp:170-275, :292-376): it binds the input
matrices, sizes the outputs (left uninitialised, as the reference does) and
calls the hooks.

PyTorch is used for device memory and the HIP stream only; no arithmetic on the
path is done by torch, and there is no fallback when the library is missing.
"""
import functools
import operator

import numpy as np
import torch

from . import capi
from .capi import LBN_STATS_REFERENCE_ORDER, LBN_STATS_SUMSQ, LBN_STATS_TWO_PASS, LbnError, call  # noqa: F401


def _prod(xs):
    return functools.reduce(operator.mul, xs, 1)


class DeviceMatrix:
    """Column-major matrix in device memory: Height/Width/LDim/Buffer of El::Matrix<T,GPU>.

    Backed by a torch tensor of shape (width, ldim); element (r, c) is tensor[c, r].
    """

    def __init__(self, height, width, dtype=torch.float32, ldim=None, device="cuda", fill=None):
        self.height, self.width = int(height), int(width)
        self.ldim = int(ldim) if ldim is not None else max(self.height, 1)
        assert self.ldim >= self.height
        self.tensor = torch.empty((max(self.width, 1), self.ldim), dtype=dtype, device=device)
        if fill is not None:
            self.tensor.fill_(fill)

    # El::Matrix vocabulary
    def Height(self):
        return self.height

    def Width(self):
        return self.width

    def LDim(self):
        return self.ldim

    def Buffer(self):
        return capi.vp(self.tensor.data_ptr())

    LockedBuffer = Buffer

    @property
    def dtype(self):
        return self.tensor.dtype

    @classmethod
    def from_numpy(cls, a, dtype=None, ldim=None, device="cuda"):
        """`a` has shape (height, width) (any memory order)."""
        a = np.asarray(a)
        h, w = a.shape
        tdt = dtype or {np.dtype("float32"): torch.float32, np.dtype("float16"): torch.float16,
                        np.dtype("float64"): torch.float64}[a.dtype]
        m = cls(h, w, dtype=tdt, ldim=ldim, device=device)
        if ldim is not None and ldim > h:
            m.tensor.fill_(float("nan"))  # padding rows must never be read or matter
        if w > 0 and h > 0:
            m.tensor[:w, :h] = torch.from_numpy(np.ascontiguousarray(a.T)).to(device=device, dtype=tdt)
        return m

    def to_numpy(self):
        """Returns an (height, width) array.  Results are consumed here: a wait between
        workgroups that ran out in any call since the last check raises ClusterWaitTimedOut."""
        check_cluster_waits()
        t = self.tensor[: self.width, : self.height]
        if t.dtype == torch.float16:
            t = t.float()
        return np.asfortranarray(t.cpu().numpy().T)


class _Vector:
    """Weights / gradient vector in device memory (fp32; binary64 for a layer of doubles)."""

    def __init__(self, n, device="cuda", values=None, dtype=torch.float32):
        if values is None:
            self.tensor = torch.empty(max(int(n), 1), dtype=dtype, device=device)
        else:
            npdt = np.float64 if dtype == torch.float64 else np.float32
            self.tensor = torch.as_tensor(np.asarray(values, dtype=npdt)).to(device).contiguous()
        self.n = int(n)

    def Buffer(self):
        return capi.vp(self.tensor.data_ptr())

    def to_numpy(self):
        check_cluster_waits()
        return self.tensor[: self.n].cpu().numpy()


def _stream():
    return capi.vp(torch.cuda.current_stream().cuda_stream)


def _null():
    return capi.vp(None)


class ClusterWaitTimedOut(LbnError):
    """A kernel in which workgroups wait for each other gave up on a wait (the sticky error
    word of a workspace is raised): the results of that call are undefined."""

    def __init__(self, where):
        RuntimeError.__init__(self, f"a bounded wait between workgroups ran out ({where}); "
                                    "results of that call are undefined")
        self.status = None


# Workspaces handed to a compute call since the last check: their error words are read where
# results are consumed (DeviceMatrix.to_numpy, which waits for the device anyway), so that a
# wait that ran out surfaces as an exception instead of as silently wrong numbers.  With
# LBN_CHECK_CLUSTER_WAITS=1 in the environment every fp_compute()/bp_compute() checks its own
# workspace right after the call (this synchronises: a debugging mode).
_PENDING = {}
_CHECK_EVERY_CALL = bool(int(__import__("os").environ.get("LBN_CHECK_CLUSTER_WAITS", "0") or 0))


def check_cluster_waits():
    """Raises ClusterWaitTimedOut if any workspace used since the last check has its error
    word raised; clears the word, so that the next use of the workspace starts clean."""
    pending = list(_PENDING.values())
    _PENDING.clear()
    for ws in pending:
        if ws.buf is None:
            continue
        flag = capi.cint(0)
        call("lbn_workspace_timed_out", _stream(), capi.vp(ws.buf.data_ptr()), flag)
        if flag.value:
            ws.buf[:64].zero_()
            raise ClusterWaitTimedOut(f"workspace of {ws.owner}")


def _after_call():
    """The debugging mode's check after a compute call.  It waits for the device, which a stream
    that is being captured into a HIP graph does not allow: calls recorded into a graph are
    checked where their results are consumed, like every call outside the debugging mode."""
    if _CHECK_EVERY_CALL and not torch.cuda.is_current_stream_capturing():
        check_cluster_waits()


class _Workspace:
    """Scratch memory owned by a layer, grown on demand (never shrunk).  The first 64 bytes
    (the error word of the kernels that wait across workgroups) are cleared when the memory
    is allocated: recycled device memory may hold anything."""

    def __init__(self, owner="a layer", header=True):
        self.buf = None
        self.owner = owner
        self.header = header  # False: scratch of a layer none of whose kernels wait across workgroups

    def get(self, nbytes, device):
        nbytes = int(nbytes)
        if nbytes == 0:
            return _null(), 0
        if self.buf is None or self.buf.numel() < nbytes:
            self.buf = torch.empty(max(nbytes, 64), dtype=torch.uint8, device=device)
            self.buf[:64].zero_()
        if self.header:
            _PENDING[id(self)] = self
        return capi.vp(self.buf.data_ptr()), nbytes


class _Layer:
    """Members every data_type_layer hands to its compute hooks."""

    def __init__(self, device="cuda"):
        self.device = device
        self.prev_activations = None    # input x
        self.activations = None         # output y
        self.prev_error_signals = None  # dL/dy
        self.error_signals = None       # dL/dx
        self._ws = _Workspace(type(self).__name__)

    # what fp_setup_inputs/outputs and bp_setup_gradient_wrt_inputs do
    def bind_forward(self, x, in_place=False):
        self.prev_activations = x
        if in_place:
            self.activations = x
        else:
            self.activations = DeviceMatrix(x.height, x.width, dtype=x.dtype, ldim=x.ldim, device=self.device)

    def bind_backward(self, dy, in_place=False):
        self.prev_error_signals = dy
        if in_place:
            self.error_signals = dy
        else:
            self.error_signals = DeviceMatrix(dy.height, dy.width, dtype=dy.dtype, ldim=dy.ldim, device=self.device)

    # fp_call()/bp_call() return (entry point name, argument tuple) of the C-ABI call
    # that is the body of the reference's fp_compute()/bp_compute().
    def fp_compute(self):
        name, args = self.fp_call()
        call(name, *args)
        _after_call()

    def bp_compute(self):
        name, args = self.bp_call()
        call(name, *args)
        _after_call()

    def forward(self, x, in_place=False):
        self.bind_forward(x, in_place)
        self.fp_compute()
        return self.activations

    def backward(self, dy, in_place=False):
        self.bind_backward(dy, in_place)
        self.bp_compute()
        return self.error_signals


class layer_norm_layer(_Layer):
    """lbann::layer_norm_layer (include/lbann/layers/regularizers/layer_norm.hpp:53-143)."""

    def __init__(self, dims, epsilon=1e-5, scale=False, bias=False, start_dim=0,
                 scale_values=None, bias_values=None, stats_mode=LBN_STATS_TWO_PASS, device="cuda",
                 datatype=torch.float32):
        """datatype: the reference's TensorDataType; torch.float64 selects the _f64 entry points
        (weights, statistics and their gradients are then doubles as well)."""
        super().__init__(device)
        self.datatype = wt = torch.float64 if datatype == torch.float64 else torch.float32
        self.dims = tuple(int(d) for d in dims)
        self.m_epsilon, self.m_scale, self.m_bias, self.m_start_dim = float(epsilon), bool(scale), bool(bias), int(start_dim)
        sd = self.m_start_dim if self.m_start_dim >= 0 else len(self.dims) + self.m_start_dim
        if sd < 0 or sd >= len(self.dims):
            raise ValueError(f"layer norm start dimension {start_dim} does not match tensor dimensionality {len(self.dims)}")
        # get_normdims (layer_norm.hpp:362-405)
        self.num_normalized = _prod(self.dims[:sd])
        self.normalization_size = _prod(self.dims[sd:])
        self.normalization_stride = self.normalization_size
        n = self.normalization_size
        self.weights = []
        if self.m_scale:
            self.weights.append(_Vector(n, device, scale_values if scale_values is not None else np.ones(n), wt))
        if self.m_bias:
            self.weights.append(_Vector(n, device, bias_values if bias_values is not None else np.zeros(n), wt))
        self.m_scale_gradient = _Vector(n, device, dtype=wt) if self.m_scale else None
        self.m_bias_gradient = _Vector(n, device, dtype=wt) if self.m_bias else None
        self.m_statistics = None
        self.m_statistics_gradient = None
        self.stats_mode = stats_mode

    def _suffix(self):
        if self.datatype == torch.float64:
            return "f64"
        return "f16" if self.prev_activations.dtype == torch.float16 else "f32"

    def _scratch(self):
        """One scratch buffer for both directions, sized for the larger need, so that neither
        call's bound pointer is invalidated by the other growing it."""
        x = self.prev_activations
        G, n = self.num_normalized, self.normalization_size
        esize = 2 if x.dtype == torch.float16 else 4
        lib = capi.lib()
        if self.datatype == torch.float64:
            self._ws.header = False
            return self._ws.get(lib.lbn_layer_norm_bwd_workspace_bytes_f64(G, n, x.width, int(self.m_scale or self.m_bias)),
                                self.device)
        need = max(lib.lbn_layer_norm_fwd_workspace_bytes(G, n, x.width, esize),
                   lib.lbn_layer_norm_bwd_workspace_bytes(G, n, x.width, int(self.m_scale or self.m_bias), esize))
        return self._ws.get(need, self.device)

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        G, n = self.num_normalized, self.normalization_size
        if self.m_statistics is None or self.m_statistics.width != x.width:
            self.m_statistics = DeviceMatrix(2 * G, x.width, dtype=self.datatype, device=self.device)
        scale = self.weights[0].Buffer() if self.m_scale else _null()
        bias = self.weights[-1].Buffer() if self.m_bias else _null()
        ws, nb = self._scratch()
        if self.datatype == torch.float64:  # no forward scratch
            return ("lbn_layer_norm_fwd_f64",
                    (_stream(), G, n, self.normalization_stride, x.width,
                     self.m_epsilon, x.Buffer(), x.ldim, y.Buffer(), y.ldim, self.m_statistics.Buffer(),
                     self.m_statistics.ldim, scale, bias, self.stats_mode))
        return (f"lbn_layer_norm_fwd_{self._suffix()}",
                (_stream(), G, n, self.normalization_stride, x.width,
                 self.m_epsilon, x.Buffer(), x.ldim, y.Buffer(), y.ldim, self.m_statistics.Buffer(),
                 self.m_statistics.ldim, scale, bias, ws, nb, self.stats_mode))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        G, n = self.num_normalized, self.normalization_size
        if self.m_statistics_gradient is None or self.m_statistics_gradient.width != x.width:
            self.m_statistics_gradient = DeviceMatrix(2 * G, x.width, dtype=self.datatype, device=self.device)
        scale = self.weights[0].Buffer() if self.m_scale else _null()
        dscale = self.m_scale_gradient.Buffer() if self.m_scale else _null()
        dbias = self.m_bias_gradient.Buffer() if self.m_bias else _null()
        ws, nb = self._scratch()
        return (f"lbn_layer_norm_bwd_{self._suffix()}",
                (_stream(), G, n, self.normalization_stride, x.width,
                 self.m_epsilon, x.Buffer(), x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim,
                 self.m_statistics.Buffer(), self.m_statistics.ldim, self.m_statistics_gradient.Buffer(),
                 self.m_statistics_gradient.ldim, scale, dscale, dbias, ws, nb))


class instance_norm_layer(_Layer):
    """lbann::instance_norm_layer (include/lbann/layers/regularizers/instance_norm.hpp):
    channels = leading output dimension, every (sample, channel) slab normalised on its own."""

    def __init__(self, dims, epsilon=1e-5, device="cuda"):
        super().__init__(device)
        self.dims = tuple(int(d) for d in dims)
        self.m_epsilon = float(epsilon)
        self.num_channels = self.dims[0]
        self.channel_size = _prod(self.dims) // self.num_channels
        self.m_workspace = None  # (2*channels x width): means, then variances
        self._ws_fwd = _Workspace("instance_norm_layer (forward)")  # forward scratch of its own: backward's holds the statistics gradients

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        if self.m_workspace is None or self.m_workspace.width != x.width:
            self.m_workspace = DeviceMatrix(2 * self.num_channels, x.width, device=self.device)
        ws, nb = self._ws_fwd.get(capi.lib().lbn_instance_norm_fwd_workspace_bytes(
            self.num_channels, self.channel_size, x.width), self.device)
        return ("lbn_instance_norm_fwd_f32",
                (_stream(), self.num_channels, self.channel_size, x.width, self.m_epsilon, x.Buffer(),
                 x.ldim, y.Buffer(), y.ldim, self.m_workspace.Buffer(), self.m_workspace.ldim, ws, nb))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        ws, nb = self._ws.get(capi.lib().lbn_instance_norm_bwd_workspace_bytes(
            self.num_channels, self.channel_size, x.width), self.device)
        return ("lbn_instance_norm_bwd_f32",
                (_stream(), self.num_channels, self.channel_size, x.width, self.m_epsilon, x.Buffer(),
                 x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim, self.m_workspace.Buffer(),
                 self.m_workspace.ldim, ws, nb))


class entrywise_batch_normalization_layer(_Layer):
    """lbann::entrywise_batch_normalization_layer
    (include/lbann/layers/regularizers/entrywise_batch_normalization.hpp): per-entry statistics
    over the mini-batch; weights[0] running mean, weights[1] running variance.

    `comm_allreduce(matrix)` stands for the reference's comm.allreduce over the mini-batch's
    ranks (entrywise_batch_normalization.cpp:97-100, :301-303): when given, it is called on the
    (height x 2) matrix of local sums, which it must replace by their sum over the ranks, and
    `statistics_count` is the global mini-batch size (input.Width() there); the layer then
    runs the split entry points around it."""

    def __init__(self, dims, decay=0.9, epsilon=1e-5, device="cuda", comm_allreduce=None, statistics_count=None):
        super().__init__(device)
        self.dims = tuple(int(d) for d in dims)
        self.m_decay, self.m_epsilon = float(decay), float(epsilon)
        self.comm_allreduce, self.statistics_count = comm_allreduce, statistics_count
        h = _prod(self.dims)
        # default weights (entrywise_batch_normalization.hpp:159-176): mean 0, variance 1
        self.weights = [_Vector(h, device, np.zeros(h)), _Vector(h, device, np.ones(h))]
        self.m_batch_statistics = DeviceMatrix(h, 2, device=device)
        self.m_batch_statistics_gradient = DeviceMatrix(h, 2, device=device)
        self.training = True
        self._ws = _Workspace(type(self).__name__, header=False)  # partial sums only: no kernel of this layer waits

    def _scratch(self):
        x = self.prev_activations
        return self._ws.get(capi.lib().lbn_entrywise_batch_norm_workspace_bytes(x.height, x.width), self.device)

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        st = self.m_batch_statistics
        ws, nb = self._scratch()
        return ("lbn_entrywise_batch_norm_fwd_f32",
                (_stream(), x.height, x.width, self.m_decay, self.m_epsilon, int(self.training), x.Buffer(),
                 x.ldim, y.Buffer(), y.ldim, st.Buffer(), st.ldim, self.weights[0].Buffer(),
                 self.weights[1].Buffer(), ws, nb))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        st, sg = self.m_batch_statistics, self.m_batch_statistics_gradient
        ws, nb = self._scratch()
        return ("lbn_entrywise_batch_norm_bwd_f32",
                (_stream(), x.height, x.width, self.m_epsilon, int(self.training), x.Buffer(), x.ldim,
                 dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim, st.Buffer(), st.ldim, sg.Buffer(), sg.ldim,
                 self.weights[1].Buffer(), ws, nb))

    def _col(self, m, j):
        return capi.vp(m.tensor.data_ptr() + 4 * j * m.ldim)

    def fp_compute(self):
        if self.comm_allreduce is None:
            return super().fp_compute()
        x, y, st = self.prev_activations, self.activations, self.m_batch_statistics
        if self.training:
            count = int(self.statistics_count if self.statistics_count is not None else x.width)
            call("lbn_entrywise_batch_norm_fwd_sums_f32", _stream(), x.height, x.width, x.Buffer(), x.ldim,
                 st.Buffer(), st.ldim)
            self.comm_allreduce(st)
            call("lbn_entrywise_batch_norm_fwd_stats_f32", _stream(), x.height, count, self.m_decay, st.Buffer(),
                 st.ldim, self.weights[0].Buffer(), self.weights[1].Buffer())
            mean, var = self._col(st, 0), self._col(st, 1)
        else:
            mean, var = self.weights[0].Buffer(), self.weights[1].Buffer()
        call("lbn_entrywise_batch_norm_fwd_apply_f32", _stream(), x.height, x.width, self.m_epsilon, x.Buffer(), x.ldim,
             y.Buffer(), y.ldim, mean, var)

    def bp_compute(self):
        if self.comm_allreduce is None or not self.training:
            return super().bp_compute()
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        st, sg = self.m_batch_statistics, self.m_batch_statistics_gradient
        count = int(self.statistics_count if self.statistics_count is not None else x.width)
        if count > 1:
            call("lbn_entrywise_batch_norm_bwd_sums_f32", _stream(), x.height, x.width, self.m_epsilon, x.Buffer(),
                 x.ldim, dy.Buffer(), dy.ldim, st.Buffer(), st.ldim, sg.Buffer(), sg.ldim)
            self.comm_allreduce(sg)
        call("lbn_entrywise_batch_norm_bwd_apply_f32", _stream(), x.height, x.width, count, self.m_epsilon, x.Buffer(),
             x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim, st.Buffer(), st.ldim, sg.Buffer(), sg.ldim)


class batch_normalization_layer(_Layer):
    """lbann::batch_normalization_layer (include/lbann/layers/regularizers/batch_normalization.hpp:130-199),
    local statistics (statistics_group_size == 1)."""

    def __init__(self, dims, decay=0.9, epsilon=1e-5, bessel_correction=True, scale_values=None,
                 bias_values=None, stats_mode=LBN_STATS_TWO_PASS, device="cuda", datatype=torch.float32):
        super().__init__(device)
        self.datatype = wt = torch.float64 if datatype == torch.float64 else torch.float32
        self.dims = tuple(int(d) for d in dims)
        self.m_decay, self.m_epsilon, self.m_bessel_correction = float(decay), float(epsilon), bool(bessel_correction)
        self.num_channels = self.dims[0]
        self.channel_size = _prod(self.dims[1:])
        C = self.num_channels
        # weights 0..3: scale, bias, running mean, running variance (defaults 1, 0, 0, 1)
        self.weights = [
            _Vector(C, device, scale_values if scale_values is not None else np.ones(C), wt),
            _Vector(C, device, bias_values if bias_values is not None else np.zeros(C), wt),
            _Vector(C, device, np.zeros(C), wt),
            _Vector(C, device, np.ones(C), wt),
        ]
        # m_mean_and_var / m_mean_and_var_gradient: C x 2, column 0 mean, column 1 variance
        self.m_mean_and_var = DeviceMatrix(C, 2, dtype=wt, device=device)
        self.m_mean_and_var_gradient = DeviceMatrix(C, 2, dtype=wt, device=device)
        self.m_scale_gradient = _Vector(C, device, dtype=wt)
        self.m_bias_gradient = _Vector(C, device, dtype=wt)
        self.training = True
        self.stats_mode = stats_mode

    def _col(self, m, j):
        return capi.vp(m.tensor.data_ptr() + m.tensor.element_size() * j * m.ldim)

    def _scratch(self, width):
        C, cs = self.num_channels, self.channel_size
        if self.datatype == torch.float64:
            self._ws.header = False
            return self._ws.get(capi.lib().lbn_batch_norm_workspace_bytes_f64(C, cs, width), self.device)
        return self._ws.get(capi.lib().lbn_batch_norm_workspace_bytes(C, cs, width), self.device)

    def _suffix(self, x):
        if self.datatype == torch.float64:
            return "f64"
        return "f16" if x.dtype == torch.float16 else "f32"

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        C, cs = self.num_channels, self.channel_size
        ws, nb = self._scratch(x.width)
        return (f"lbn_batch_norm_fwd_{self._suffix(x)}",
                (_stream(), C, cs, x.width, int(self.m_bessel_correction),
                 self.m_epsilon, self.m_decay, int(self.training), x.Buffer(), x.ldim, y.Buffer(), y.ldim,
                 self._col(self.m_mean_and_var, 0), self._col(self.m_mean_and_var, 1),
                 self.weights[0].Buffer(), self.weights[1].Buffer(), self.weights[2].Buffer(),
                 self.weights[3].Buffer(), ws, nb, self.stats_mode))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        C, cs = self.num_channels, self.channel_size
        ws, nb = self._scratch(x.width)
        name = f"lbn_batch_norm_bwd_{self._suffix(x)}"
        if self.stats_mode & LBN_STATS_REFERENCE_ORDER and self.datatype != torch.float64:  # parity tests: the reference's order of summation
            name = "lbn_batch_norm_bwd_reference_order_f32"
        return (name,
                (_stream(), C, cs, x.width, int(self.m_bessel_correction),
                 self.m_epsilon, int(self.training), x.Buffer(), x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(),
                 dx.ldim, self._col(self.m_mean_and_var, 0), self._col(self.m_mean_and_var, 1),
                 self.weights[2].Buffer(), self.weights[3].Buffer(), self.weights[0].Buffer(),
                 self.m_scale_gradient.Buffer(), self.m_bias_gradient.Buffer(),
                 self._col(self.m_mean_and_var_gradient, 0), self._col(self.m_mean_and_var_gradient, 1), ws, nb))


class _softmax_like(_Layer):
    _name = None

    @staticmethod
    def _suffix(m):
        return {torch.float16: "f16", torch.float64: "f64"}.get(m.dtype, "f32")

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        if x.dtype == torch.float64:  # TensorDataType = double: no scratch
            return (f"lbn_{self._name}_fwd_f64", (_stream(), x.height, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim))
        ws, nb = self._ws.get(capi.lib().lbn_softmax_workspace_bytes(x.height, x.width), self.device)
        return (f"lbn_{self._name}_fwd_{self._suffix(x)}",
                (_stream(), x.height, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim, ws, nb))

    def bp_call(self):
        y, dy, dx = self.activations, self.prev_error_signals, self.error_signals
        if y.dtype == torch.float64:
            return (f"lbn_{self._name}_bwd_f64",
                    (_stream(), y.height, y.width, y.Buffer(), y.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim))
        ws, nb = self._ws.get(capi.lib().lbn_softmax_workspace_bytes(y.height, y.width), self.device)
        return (f"lbn_{self._name}_bwd_{self._suffix(y)}",
                (_stream(), y.height, y.width, y.Buffer(), y.ldim, dy.Buffer(), dy.ldim, dx.Buffer(),
                 dx.ldim, ws, nb))


class softmax_layer(_softmax_like):
    """lbann::softmax_layer, data-parallel layout, softmax_mode::INSTANCE
    (include/lbann/layers/activations/softmax.hpp:85-262)."""
    _name = "softmax"

    def __init__(self, mode="instance", device="cuda"):
        super().__init__(device)
        if mode != "instance":
            # the reference's CPU path rejects every other mode (openmp/softmax.hpp:61-63)
            raise ValueError("Unsupported softmax mode")


class log_softmax_layer(_softmax_like):
    """lbann::log_softmax_layer (include/lbann/layers/activations/log_softmax.hpp)."""
    _name = "log_softmax"


class channelwise_softmax_layer(_Layer):
    """lbann::channelwise_softmax_layer (include/lbann/layers/misc/channelwise_softmax.hpp:50-107)."""

    def __init__(self, dims, dim=0, single_dim_mode=False, device="cuda"):
        super().__init__(device)
        self.dims = tuple(int(d) for d in dims)
        nd = len(self.dims)
        if dim < -nd or dim >= nd:
            raise ValueError(f"Dimension {dim} is out of bounds for Channelwise Softmax layer on tensor with {nd} dimensions.")
        if not single_dim_mode and dim not in (0, -nd, nd - 1, -1):
            raise ValueError("Channelwise softmax with all dimensions is only supported for the first or last tensor dimensions.")
        self.m_dim, self.m_single_dim_mode = int(dim), bool(single_dim_mode)

    def get_channel_size_and_stride(self):
        """(channel_size, channel_stride, num_channels), channelwise_softmax_impl.hpp:58-104."""
        dims = self.dims
        d = self.m_dim + len(dims) if self.m_dim < 0 else self.m_dim
        total = _prod(dims)
        if self.m_single_dim_mode:
            cs = dims[d]
            return cs, _prod(dims[d:]), total // cs
        cs = total // dims[d]
        return cs, (cs if d == 0 else 1), dims[d]

    def fp_call(self):
        x, y = self.prev_activations, self.activations
        cs, stride, C = self.get_channel_size_and_stride()
        if x.dtype == torch.float64:
            return ("lbn_channelwise_softmax_fwd_f64",
                    (_stream(), C, cs, stride, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim))
        ws, nb = self._ws.get(capi.lib().lbn_channelwise_softmax_workspace_bytes(C, cs, x.width), self.device)
        return ("lbn_channelwise_softmax_fwd_f32",
                (_stream(), C, cs, stride, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim, ws, nb))

    def bp_call(self):
        y, dy, dx = self.activations, self.prev_error_signals, self.error_signals
        cs, stride, C = self.get_channel_size_and_stride()
        if y.dtype == torch.float64:
            return ("lbn_channelwise_softmax_bwd_f64",
                    (_stream(), C, cs, stride, y.width, y.Buffer(), y.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim))
        ws, nb = self._ws.get(capi.lib().lbn_channelwise_softmax_workspace_bytes(C, cs, y.width), self.device)
        return ("lbn_channelwise_softmax_bwd_f32",
                (_stream(), C, cs, stride, y.width, y.Buffer(), y.ldim, dy.Buffer(), dy.ldim, dx.Buffer(),
                 dx.ldim, ws, nb))


class _scale_bias_layer(_Layer):
    """Shared state of the two scale/bias layers: one weights matrix (n x 2), column 0 scale
    (default 1), column 1 bias (default 0), and m_weights_gradient of the same shape."""

    def _setup_weights(self, n, device):
        self.weights = DeviceMatrix(n, 2, device=device)
        self.weights.tensor[0].fill_(1.0)
        self.weights.tensor[1].fill_(0.0)
        self.m_weights_gradient = DeviceMatrix(n, 2, device=device)

    def set_weights(self, scale, bias):
        n = self.weights.height
        self.weights.tensor[0, :n] = torch.as_tensor(np.asarray(scale, np.float32).reshape(-1)).to(self.device)
        self.weights.tensor[1, :n] = torch.as_tensor(np.asarray(bias, np.float32).reshape(-1)).to(self.device)


class entrywise_scale_bias_layer(_scale_bias_layer):
    """lbann::entrywise_scale_bias_layer (include/lbann/layers/learning/entrywise_scale_bias.hpp:57-203)."""

    def __init__(self, dims, device="cuda"):
        super().__init__(device)
        self.dims = tuple(int(d) for d in dims)
        self._setup_weights(_prod(self.dims), device)

    def fp_call(self):
        x, y, wt = self.prev_activations, self.activations, self.weights
        return ("lbn_entrywise_scale_bias_fwd_f32",
                (_stream(), x.height, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim, wt.Buffer(), wt.ldim))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        wt, wg = self.weights, self.m_weights_gradient
        self._ws.header = False
        ws, nb = self._ws.get(capi.lib().lbn_entrywise_scale_bias_bwd_workspace_bytes(x.height, x.width),
                              self.device)
        return ("lbn_entrywise_scale_bias_bwd_f32",
                (_stream(), x.height, x.width, x.Buffer(), x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim,
                 wt.Buffer(), wt.ldim, wg.Buffer(), wg.ldim, ws, nb))


class channelwise_scale_bias_layer(_scale_bias_layer):
    """lbann::channelwise_scale_bias_layer (include/lbann/layers/learning/channelwise_scale_bias.hpp:60-206)."""

    def __init__(self, dims, device="cuda"):
        super().__init__(device)
        self.dims = tuple(int(d) for d in dims)
        self.num_channels = self.dims[0]
        self.channel_size = _prod(self.dims[1:])
        self._setup_weights(self.num_channels, device)

    def fp_call(self):
        x, y, wt = self.prev_activations, self.activations, self.weights
        return ("lbn_channelwise_scale_bias_fwd_f32",
                (_stream(), self.num_channels, self.channel_size, x.width, x.Buffer(), x.ldim, y.Buffer(), y.ldim,
                 wt.Buffer(), wt.ldim))

    def bp_call(self):
        x, dy, dx = self.prev_activations, self.prev_error_signals, self.error_signals
        wt, wg = self.weights, self.m_weights_gradient
        C, cs = self.num_channels, self.channel_size
        self._ws.header = False
        ws, nb = self._ws.get(capi.lib().lbn_channelwise_scale_bias_bwd_workspace_bytes(C, cs, x.width), self.device)
        return ("lbn_channelwise_scale_bias_bwd_f32",
                (_stream(), C, cs, x.width, x.Buffer(), x.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim,
                 wt.Buffer(), wt.ldim, wg.Buffer(), wg.ldim, ws, nb))


class cross_entropy_layer:
    """lbann::cross_entropy_layer (include/lbann/layers/loss/cross_entropy.hpp:75-190): two
    parents (prediction, ground truth), output of dims {1}.  `dims` are the prediction's
    dimensions; with use_labels the ground truth has dims (1, dims[1:]) and holds class
    indices (cross_entropy_impl.hpp:59-133)."""

    def __init__(self, dims, use_labels=False, device="cuda"):
        self.device = device
        self.dims = tuple(int(d) for d in dims)
        self.m_use_labels = bool(use_labels)
        if self.m_use_labels and len(self.dims) < 2:
            raise ValueError("cross entropy layer expects both input tensors to have the same number of "
                             "dimensions and have >2 dimensions when use_labels is enabled.")
        self.spatial_sample_size = _prod(self.dims[1:])
        self.prev_activations = [None, None]
        self.activations = None
        self.prev_error_signals = None
        self.error_signals = [None, None]
        self._ws = _Workspace("cross_entropy_layer", header=False)

    @staticmethod
    def _suffix(*matrices):
        """fp32 or fp16 storage (the reference instantiates the layer for both,
        cross_entropy.cpp:157-166); every matrix of a call has the layer's one data type."""
        kinds = {m.dtype for m in matrices if m is not None}
        if len(kinds) != 1:
            raise TypeError(f"cross entropy: matrices of different types {sorted(map(str, kinds))}")
        return "f16" if kinds.pop() == torch.float16 else "f32"

    def fp_call(self):
        x, t, y = self.prev_activations[0], self.prev_activations[1], self.activations
        ws, nb = self._ws.get(capi.lib().lbn_cross_entropy_fwd_workspace_bytes(x.height, x.width), self.device)
        return (f"lbn_cross_entropy_fwd_{self._suffix(x, t, y)}",
                (_stream(), x.height, x.width, int(self.m_use_labels), self.spatial_sample_size, x.Buffer(), x.ldim,
                 t.Buffer(), t.ldim, y.Buffer(), y.ldim, ws, nb))

    def bp_call(self):
        x, t, dy = self.prev_activations[0], self.prev_activations[1], self.prev_error_signals
        dx, dt = self.error_signals
        return (f"lbn_cross_entropy_bwd_{self._suffix(x, t, dy, dx, dt)}",
                (_stream(), x.height, x.width, int(self.m_use_labels), self.spatial_sample_size, x.Buffer(), x.ldim,
                 t.Buffer(), t.ldim, dy.Buffer(), dy.ldim, dx.Buffer(), dx.ldim,
                 dt.Buffer() if dt is not None else _null(), dt.ldim if dt is not None else 0))

    def fp_compute(self):
        name, args = self.fp_call()
        call(name, *args)
        _after_call()

    def bp_compute(self):
        name, args = self.bp_call()
        call(name, *args)
        _after_call()

    def forward(self, prediction, ground_truth):
        self.prev_activations = [prediction, ground_truth]
        self.activations = DeviceMatrix(1, prediction.width, dtype=prediction.dtype, device=self.device)
        self.fp_compute()
        return self.activations

    def backward(self, dy):
        """dy: (1 x width) gradient w.r.t. the loss.  Returns [dL/dprediction, dL/dground_truth];
        the second is None with use_labels (the reference leaves that error signal untouched)."""
        x, t = self.prev_activations
        self.prev_error_signals = dy
        self.error_signals = [DeviceMatrix(x.height, x.width, dtype=x.dtype, ldim=x.ldim, device=self.device),
                              None if self.m_use_labels else DeviceMatrix(t.height, t.width, dtype=t.dtype,
                                                                          ldim=t.ldim, device=self.device)]
        self.bp_compute()
        return self.error_signals


def softmax_cross_entropy_forward(softmax, cross_entropy, x, ground_truth):
    """Forward of a softmax_layer whose only child is a cross_entropy_layer, in one call
    (lbn_softmax_cross_entropy_fwd_f32): what softmax.forward(x) followed by
    cross_entropy.forward(y, ground_truth) computes, with both layers' members bound as
    those two calls bind them, so each layer's backward runs unchanged afterwards.
    Returns (y, loss).  fp32 storage only."""
    if x.dtype != torch.float32:
        raise TypeError("softmax_cross_entropy_forward takes fp32 matrices")
    softmax.bind_forward(x)
    y = softmax.activations
    cross_entropy.prev_activations = [y, ground_truth]
    cross_entropy.activations = DeviceMatrix(1, x.width, device=cross_entropy.device)
    loss = cross_entropy.activations
    ws, nb = softmax._ws.get(capi.lib().lbn_softmax_cross_entropy_fwd_workspace_bytes(x.height, x.width), softmax.device)
    call("lbn_softmax_cross_entropy_fwd_f32", _stream(), x.height, x.width, int(cross_entropy.m_use_labels),
         cross_entropy.spatial_sample_size, x.Buffer(), x.ldim, ground_truth.Buffer(), ground_truth.ldim,
         y.Buffer(), y.ldim, loss.Buffer(), loss.ldim, ws, nb)
    _after_call()
    return y, loss


def softmax_cross_entropy_backward(softmax, cross_entropy, dloss, want_dtruth=False):
    """Backward of the pair in one call (lbn_softmax_cross_entropy_bwd_f32): what
    cross_entropy.backward(dloss) followed by softmax.backward(dprediction) computes, without
    the gradient with respect to the prediction ever being written.  The layers must have run
    their forward (together or one after the other).  Returns dx; cross_entropy.error_signals
    becomes [None, dtruth or None]."""
    y, truth = cross_entropy.prev_activations
    if y is not softmax.activations:
        raise ValueError("the softmax layer's output is not the cross-entropy layer's prediction")
    cross_entropy.prev_error_signals = dloss
    dtruth = None
    if want_dtruth and not cross_entropy.m_use_labels:
        dtruth = DeviceMatrix(truth.height, truth.width, ldim=truth.ldim, device=cross_entropy.device)
    cross_entropy.error_signals = [None, dtruth]
    softmax.prev_error_signals = None
    softmax.error_signals = DeviceMatrix(y.height, y.width, ldim=y.ldim, device=softmax.device)
    dx = softmax.error_signals
    ws, nb = softmax._ws.get(capi.lib().lbn_softmax_workspace_bytes(y.height, y.width), softmax.device)
    call("lbn_softmax_cross_entropy_bwd_f32", _stream(), y.height, y.width, int(cross_entropy.m_use_labels),
         cross_entropy.spatial_sample_size, y.Buffer(), y.ldim, truth.Buffer(), truth.ldim, dloss.Buffer(), dloss.ldim,
         dx.Buffer(), dx.ldim, dtruth.Buffer() if dtruth is not None else _null(),
         dtruth.ldim if dtruth is not None else 0, ws, nb)
    _after_call()
    return dx


class gradient_buffer:
    """The optimizer's gradient buffer as the layers see it: optimizer::add_to_gradient and
    get_gradient_buffer (include/lbann/optimizers/optimizer_impl.hpp:207-288) with their status
    machine (include/lbann/optimizers/optimizer.hpp:54-70), for one process (RedundantSize = 1,
    so a needed synchronisation changes the status and nothing else).

    `gradient` is a (height x width) DeviceMatrix.  It starts `cleared`: the first contribution
    overwrites it without reading it, later ones accumulate."""

    READY, CLEARED, SYNC_NEEDED = "ready", "cleared", "sync_needed"

    def __init__(self, height, width=1, device="cuda"):
        self.gradient = DeviceMatrix(height, width, device=device)
        self.status = self.CLEARED

    def clear(self):
        self.status = self.CLEARED

    def _scales(self, sync_needed):
        # (buf_scale, in_scale) and the status transition of get_gradient_buffer
        if self.status == self.READY:
            if sync_needed:
                self.status = self.SYNC_NEEDED
            return 1.0, 1.0
        if self.status == self.CLEARED:
            self.status = self.SYNC_NEEDED if sync_needed else self.READY
            return 0.0, 1.0
        if self.status == self.SYNC_NEEDED:
            return 1.0, 1.0
        raise ValueError(f"unexpected gradient status ({self.status})")

    def add_to_gradient(self, contrib, scale=1.0, sync_needed=False, ldim=None):
        """contrib: a DeviceMatrix of the buffer's shape, or a _Vector / torch tensor holding one column
        (then `ldim` is its leading dimension when the buffer has several columns)."""
        g = self.gradient
        buf_scale, in_scale = self._scales(sync_needed)
        if isinstance(contrib, DeviceMatrix):
            if (contrib.height, contrib.width) != (g.height, g.width):
                raise ValueError("gradient contribution has the wrong shape")
            ptr, ld = contrib.Buffer(), contrib.ldim
        else:
            t = contrib.tensor if hasattr(contrib, "tensor") else contrib
            ld = int(ldim) if ldim is not None else g.height
            if t.numel() < (g.width - 1) * ld + g.height:
                raise ValueError("gradient contribution is too small")
            ptr = capi.vp(t.data_ptr())
        call("lbn_gradient_sink_f32", _stream(), g.height, g.width, buf_scale, in_scale * float(scale), ptr, ld,
             g.Buffer(), g.ldim)

    def finish_sync(self):
        """What the all-reduce completes on several processes; here the values are already final."""
        if self.status == self.SYNC_NEEDED:
            self.status = self.READY
