"""ctypes binding of liblbnorm.so (the C ABI declared in include/lbnorm.h).

Loading fails loudly: there is no CPU or PyTorch fallback for any entry point.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("LBN_LIB") or os.path.join(_HERE, "liblbnorm.so")

i64 = ctypes.c_int64
f32 = ctypes.c_float
f64 = ctypes.c_double
cint = ctypes.c_int
vp = ctypes.c_void_p
sz = ctypes.c_size_t

LBN_OK = 0
LBN_ERR_INVALID_ARGUMENT = -1
LBN_ERR_WORKSPACE = -2
LBN_ERR_UNSUPPORTED = -3
LBN_STATS_TWO_PASS = 0
LBN_STATS_SUMSQ = 1
LBN_STATS_REFERENCE_ORDER = 2

# name -> (restype, argtypes); mirrors include/lbnorm.h declaration by declaration
PROTOTYPES = {
    "lbn_version": (cint, []),
    "lbn_status_string": (ctypes.c_char_p, [cint]),
    "lbn_workspace_timed_out": (cint, [vp, vp, ctypes.POINTER(cint)]),
    "lbn_selftest_cluster_wait_gives_up": (cint, [vp, vp, sz, cint, vp]),
    "lbn_selftest_copy_pipeline_f32": (cint, [vp, i64, i64, i64, vp, i64, vp, i64, cint]),
    "lbn_layer_norm_fwd_workspace_bytes": (sz, [i64, i64, i64, cint]),
    "lbn_layer_norm_fwd_f32": (cint, [vp, i64, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, vp, vp, sz, cint]),
    "lbn_layer_norm_fwd_f16": (cint, [vp, i64, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, vp, vp, sz, cint]),
    "lbn_layer_norm_bwd_workspace_bytes": (sz, [i64, i64, i64, cint, cint]),
    "lbn_layer_norm_bwd_f32": (cint, [vp, i64, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, i64,
                                      vp, i64, vp, vp, vp, vp, sz]),
    "lbn_layer_norm_bwd_f16": (cint, [vp, i64, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, i64,
                                      vp, i64, vp, vp, vp, vp, sz]),
    "lbn_instance_norm_fwd_workspace_bytes": (sz, [i64, i64, i64]),
    "lbn_instance_norm_fwd_f32": (cint, [vp, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_instance_norm_bwd_workspace_bytes": (sz, [i64, i64, i64]),
    "lbn_instance_norm_bwd_f32": (cint, [vp, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_entrywise_batch_norm_workspace_bytes": (sz, [i64, i64]),
    "lbn_entrywise_batch_norm_fwd_f32": (cint, [vp, i64, i64, f32, f32, cint, vp, i64, vp, i64, vp, i64, vp, vp, vp, sz]),
    "lbn_entrywise_batch_norm_fwd_reference_order_f32": (cint, [vp, i64, i64, f32, f32, vp, i64, vp, i64, vp, i64, vp, vp]),
    "lbn_entrywise_batch_norm_bwd_f32": (cint, [vp, i64, i64, f32, cint, vp, i64, vp, i64, vp, i64, vp, i64,
                                                vp, i64, vp, vp, sz]),
    "lbn_batch_norm_workspace_bytes": (sz, [i64, i64, i64]),
    "lbn_batch_norm_fwd_f32": (cint, [vp, i64, i64, i64, cint, f32, f32, cint, vp, i64, vp, i64, vp, vp,
                                      vp, vp, vp, vp, vp, sz, cint]),
    "lbn_batch_norm_bwd_f32": (cint, [vp, i64, i64, i64, cint, f32, cint, vp, i64, vp, i64, vp, i64, vp,
                                      vp, vp, vp, vp, vp, vp, vp, vp, vp, sz]),
    "lbn_batch_norm_bwd_reference_order_f32": (cint, [vp, i64, i64, i64, cint, f32, cint, vp, i64, vp, i64, vp, i64, vp,
                                                      vp, vp, vp, vp, vp, vp, vp, vp, vp, sz]),
    "lbn_batch_norm_fwd_f16": (cint, [vp, i64, i64, i64, cint, f32, f32, cint, vp, i64, vp, i64, vp, vp,
                                      vp, vp, vp, vp, vp, sz, cint]),
    "lbn_batch_norm_bwd_f16": (cint, [vp, i64, i64, i64, cint, f32, cint, vp, i64, vp, i64, vp, i64, vp,
                                      vp, vp, vp, vp, vp, vp, vp, vp, vp, sz]),
    "lbn_batch_norm_fwd_sums_f32": (cint, [vp, i64, i64, i64, vp, i64, vp, vp, vp, sz]),
    "lbn_batch_norm_fwd_stats_f32": (cint, [vp, i64, i64, cint, f32, f32, vp, vp, vp, vp]),
    "lbn_batch_norm_fwd_apply_f32": (cint, [vp, i64, i64, i64, f32, vp, i64, vp, i64, vp, vp, vp, vp]),
    "lbn_batch_norm_bwd_sums_f32": (cint, [vp, i64, i64, i64, f32, vp, i64, vp, i64, vp, vp, vp, vp, vp,
                                           vp, vp, vp, sz]),
    "lbn_batch_norm_bwd_apply_f32": (cint, [vp, i64, i64, i64, i64, cint, f32, vp, i64, vp, i64, vp, i64,
                                            vp, vp, vp, vp, vp]),
    "lbn_softmax_workspace_bytes": (sz, [i64, i64]),
    "lbn_softmax_fwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_bwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_fwd_reference_order_f32": (cint, [vp, i64, i64, vp, i64, vp, i64]),
    "lbn_log_softmax_bwd_reference_order_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_softmax_fwd_static_scratch_max_bytes": (sz, []),
    "lbn_softmax_fwd_static_scratch_f32": (cint, [vp, i64, i64, vp, i64, vp, i64]),
    "lbn_softmax_fwd_static_scratch_prepare": (cint, []),
    "lbn_softmax_fwd_static_scratch_timed_out": (cint, [vp, ctypes.POINTER(ctypes.c_int)]),
    "lbn_log_softmax_fwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_log_softmax_bwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_fwd_f16": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_bwd_f16": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_log_softmax_fwd_f16": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_log_softmax_bwd_f16": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_channelwise_softmax_workspace_bytes": (sz, [i64, i64, i64]),
    "lbn_channelwise_softmax_fwd_f32": (cint, [vp, i64, i64, i64, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_channelwise_softmax_bwd_f32": (cint, [vp, i64, i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_cross_entropy_fwd_workspace_bytes": (sz, [i64, i64]),
    "lbn_softmax_cross_entropy_fwd_f32": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_softmax_cross_entropy_bwd_f32": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_cross_entropy_fwd_workspace_bytes": (sz, [i64, i64]),
    "lbn_cross_entropy_fwd_f32": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_cross_entropy_bwd_f32": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_cross_entropy_fwd_f16": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_cross_entropy_bwd_f16": (cint, [vp, i64, i64, cint, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_entrywise_scale_bias_fwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_entrywise_scale_bias_bwd_workspace_bytes": (sz, [i64, i64]),
    "lbn_entrywise_scale_bias_bwd_f32": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, sz]),
    "lbn_channelwise_scale_bias_fwd_f32": (cint, [vp, i64, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_channelwise_scale_bias_bwd_workspace_bytes": (sz, [i64, i64, i64]),
    "lbn_channelwise_scale_bias_bwd_f32": (cint, [vp, i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, i64, vp, i64,
                                                  vp, sz]),
    "lbn_entrywise_batch_norm_fwd_sums_f32": (cint, [vp, i64, i64, vp, i64, vp, i64]),
    "lbn_entrywise_batch_norm_fwd_stats_f32": (cint, [vp, i64, i64, f32, vp, i64, vp, vp]),
    "lbn_entrywise_batch_norm_fwd_apply_f32": (cint, [vp, i64, i64, f32, vp, i64, vp, i64, vp, vp]),
    "lbn_entrywise_batch_norm_bwd_sums_f32": (cint, [vp, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_entrywise_batch_norm_bwd_apply_f32": (cint, [vp, i64, i64, i64, f32, vp, i64, vp, i64, vp, i64, vp, i64,
                                                      vp, i64]),
    "lbn_gradient_sink_f32": (cint, [vp, i64, i64, f32, f32, vp, i64, vp, i64]),
    "lbn_softmax_fwd_f64": (cint, [vp, i64, i64, vp, i64, vp, i64]),
    "lbn_softmax_bwd_f64": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_log_softmax_fwd_f64": (cint, [vp, i64, i64, vp, i64, vp, i64]),
    "lbn_log_softmax_bwd_f64": (cint, [vp, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_channelwise_softmax_fwd_f64": (cint, [vp, i64, i64, i64, i64, vp, i64, vp, i64]),
    "lbn_channelwise_softmax_bwd_f64": (cint, [vp, i64, i64, i64, i64, vp, i64, vp, i64, vp, i64]),
    "lbn_layer_norm_fwd_f64": (cint, [vp, i64, i64, i64, i64, f64, vp, i64, vp, i64, vp, i64, vp, vp, cint]),
    "lbn_layer_norm_bwd_workspace_bytes_f64": (sz, [i64, i64, i64, cint]),
    "lbn_layer_norm_bwd_f64": (cint, [vp, i64, i64, i64, i64, f64, vp, i64, vp, i64, vp, i64, vp, i64,
                                      vp, i64, vp, vp, vp, vp, sz]),
    "lbn_batch_norm_workspace_bytes_f64": (sz, [i64, i64, i64]),
    "lbn_batch_norm_fwd_f64": (cint, [vp, i64, i64, i64, cint, f64, f64, cint, vp, i64, vp, i64, vp, vp,
                                      vp, vp, vp, vp, vp, sz, cint]),
    "lbn_batch_norm_bwd_f64": (cint, [vp, i64, i64, i64, cint, f64, cint, vp, i64, vp, i64, vp, i64, vp,
                                      vp, vp, vp, vp, vp, vp, vp, vp, vp, sz]),
}

_lib = None


class LbnError(RuntimeError):
    """A non-zero status returned through the C ABI (the adapter's thrown error)."""

    def __init__(self, fn, status, text):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m lbann_amd.build` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def call(name, *args):
    """Calls a status-returning entry point and raises LbnError on a non-zero status."""
    status = getattr(lib(), name)(*args)
    if status != 0:
        raise LbnError(name, status, lib().lbn_status_string(status).decode())
    return status
