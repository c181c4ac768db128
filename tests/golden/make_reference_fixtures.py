"""Regenerates tests/golden/reference_unit_tests.npz.

The reference holds no golden files for the normalization / softmax layers: each of
its layer tests draws a seeded NumPy dataset inside the test file, evaluates a
float64 NumPy closed form, and lets the framework's forward result deviate from
it by a stated tolerance.  This script re-creates those datasets (same legacy
`np.random.seed` stream, same draw order, same shapes) and stores, for each,
the inputs and the float64 closed-form expectation together with the tolerance
the reference test states.  Nothing from the reference is imported or run;
the formulas below are the textbook definitions the reference tests also use.

Datasets and tolerances (reference file:line):
  layer_norm            ci_test/unit_tests/test_unit_layer_layer_norm.py:21-24, :38-43, :107-113
  layer_norm (affine)   ci_test/unit_tests/test_unit_layer_layernorm_affine.py:7-15, :67-104
  layer_norm (multidim) ci_test/unit_tests/test_unit_layer_layernorm_affine.py:40-61
  batch_normalization   ci_test/unit_tests/test_unit_layer_batch_normalization.py:21-25 (no forward pin there)
  softmax               ci_test/unit_tests/test_unit_layer_softmax.py:21-24, :38-48
  log_softmax           ci_test/unit_tests/test_unit_layer_log_softmax.py:21-24, :38-48
  channelwise_softmax   ci_test/unit_tests/test_unit_layer_channelwise_softmax.py:21-26, :47-54, :109-137
  instance_norm         ci_test/unit_tests/test_unit_layer_instance_norm.py:21-24, :38-44
  entrywise_batch_norm  ci_test/unit_tests/test_unit_layer_entrywise_batch_normalization.py:21-25
                        (no forward pin there: gradient check only)
  cross_entropy         ci_test/unit_tests/test_unit_layer_cross_entropy.py:29-36, :53-76, :147-164,
                        :192-209
  entrywise_scale_bias  ci_test/unit_tests/test_unit_layer_entrywise_scale_bias.py:21-27, :98-110
  channelwise_scale_bias ci_test/unit_tests/test_unit_layer_channelwise_scale_bias.py:21-27, :90-103

Run:  python tests/golden/make_reference_fixtures.py
"""
import os

import numpy as np

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_unit_tests.npz")


def l2norm2_metric(y):
    """Mean over samples (axis 0) of the squared L2 norm, float64."""
    y = np.asarray(y, dtype=np.float64).reshape(y.shape[0], -1)
    return float(np.mean(np.sum(y * y, axis=1)))


def main():
    fx = {}

    # ---- layer norm, whole sample, no affine, eps 1e-5
    np.random.seed(20191114)
    x = np.random.normal(size=(31, 31)).astype(np.float32)
    xd = x.astype(np.float64)
    mu = xd.mean(axis=1, keepdims=True)
    var = xd.var(axis=1, ddof=0, keepdims=True)
    y = (xd - mu) / np.sqrt(var + 1e-5)
    fx["ln_x"] = x
    fx["ln_y"] = y
    fx["ln_metric"] = np.float64(l2norm2_metric(y))

    # ---- layer norm with scale / bias.  The reference's NumPy expectation divides by
    # (std + eps) instead of sqrt(var + eps); its test accepts a mean squared error of
    # 1e-8, so both expectations are stored: the exact one and the one the test holds.
    np.random.seed(20230814)
    x = np.random.normal(size=(31, 31)).astype(np.float32)
    scale = np.random.rand(31).astype(np.float32)
    bias = np.random.rand(31).astype(np.float32)
    xd = x.astype(np.float64)
    mu = xd.mean(axis=1, keepdims=True)
    var = xd.var(axis=1, ddof=0, keepdims=True)
    fx["lna_x"] = x
    fx["lna_scale"] = scale
    fx["lna_bias"] = bias
    fx["lna_y_exact"] = (xd - mu) / np.sqrt(var + 1e-5) * scale.astype(np.float64) + bias.astype(np.float64)
    x32mu = x.mean(axis=-1, keepdims=True)
    x32sd = x.std(axis=-1, ddof=0, keepdims=True)
    fx["lna_y_test_scaled_bias"] = (x - x32mu) / (x32sd + 1e-5) * scale + bias
    fx["lna_y_test_scaled"] = (x - x32mu) / (x32sd + 1e-5) * scale
    fx["lna_y_test_plain"] = (x - x32mu) / (x32sd + 1e-5)

    # ---- layer norm over trailing dims of a (31,2,5) sample, start_dim in {-1, 1, 0}
    np.random.seed(20230814)
    x = np.random.rand(31, 31, 2, 5).astype(np.float32)
    fx["lnm_x"] = x
    for start_dim, axes in ((-1, (3,)), (1, (2, 3)), (0, (1, 2, 3))):
        m = x.mean(axis=axes, keepdims=True)
        s = x.std(axis=axes, ddof=0, keepdims=True)
        fx[f"lnm_y_test_sd{start_dim}"] = (x - m) / (s + 1e-5)
        xd = x.astype(np.float64)
        md = xd.mean(axis=axes, keepdims=True)
        vd = xd.var(axis=axes, ddof=0, keepdims=True)
        fx[f"lnm_y_exact_sd{start_dim}"] = (xd - md) / np.sqrt(vd + 1e-5)

    # ---- batch norm dataset (the reference pins only gradients on it); the stored
    # expectation is the training-mode definition in float64: per-channel statistics
    # over batch and spatial positions, variance scaled by n/(n-1), clamped below at
    # eps and then eps added again under the square root, gamma=1, beta=0.
    np.random.seed(20200827)
    x = np.random.normal(size=(29, 7 * 5 * 3)).astype(np.float32)
    fx["bn_x"] = x
    for tag, batch in (("mb14", x[:14]), ("all29", x)):
        xd = batch.astype(np.float64).reshape(batch.shape[0], 7, 15)
        n = xd.shape[0] * 15
        mean = xd.mean(axis=(0, 2))
        var_b = xd.var(axis=(0, 2), ddof=0)
        for bessel in (0, 1):
            var = np.maximum(var_b * n / (n - bessel), 1e-5)
            yb = (xd - mean[None, :, None]) / np.sqrt(var[None, :, None] + 1e-5)
            fx[f"bn_{tag}_b{bessel}_mean"] = mean
            fx[f"bn_{tag}_b{bessel}_var"] = var
            fx[f"bn_{tag}_b{bessel}_y"] = yb.reshape(batch.shape[0], -1)

    # ---- softmax
    np.random.seed(201910142)
    x = np.random.normal(size=(19, 7)).astype(np.float32)
    xd = x.astype(np.float64)
    e = np.exp(xd - xd.max(axis=1, keepdims=True))
    y = e / e.sum(axis=1, keepdims=True)
    fx["sm_x"] = x
    fx["sm_y"] = y
    fx["sm_metric"] = np.float64(l2norm2_metric(y))

    # ---- log-softmax
    np.random.seed(201910213)
    x = np.random.normal(size=(15, 11)).astype(np.float32)
    xd = x.astype(np.float64)
    sh = xd - xd.max(axis=1, keepdims=True)
    y = sh - np.log(np.exp(sh).sum(axis=1, keepdims=True))
    fx["lsm_x"] = x
    fx["lsm_y"] = y
    fx["lsm_metric"] = np.float64(l2norm2_metric(y))

    # ---- channelwise softmax on (5,2,7) samples: default mode (softmax over the
    # trailing (2,7) slab of each of 5 channels) and single-dim mode on the last axis.
    np.random.seed(20200115)
    x = np.random.normal(loc=0.5, size=(15, 5 * 2 * 7)).astype(np.float32)
    fx["cws_x"] = x
    xd = x.astype(np.float64).reshape(15, 5, 2, 7)
    for tag, axes in (("default", (2, 3)), ("lastdim", (3,))):
        e = np.exp(xd - xd.max(axis=axes, keepdims=True))
        y = e / e.sum(axis=axes, keepdims=True)
        fx[f"cws_y_{tag}"] = y.reshape(15, -1)
        fx[f"cws_metric_{tag}"] = np.float64(l2norm2_metric(y))

    # ---- instance norm on (5,3,7) samples: per (sample, channel) statistics over the
    # trailing (3,7) slab, biased variance, eps 1e-5, no affine.
    np.random.seed(20200107)
    x = np.random.normal(loc=0.5, size=(15, 5 * 3 * 7)).astype(np.float32)
    xd = x.astype(np.float64).reshape(15, 5, 3, 7)
    mean = xd.mean(axis=(2, 3), keepdims=True)
    var = xd.var(axis=(2, 3), ddof=0, keepdims=True)
    y = (xd - mean) / np.sqrt(var + 1e-5)
    fx["in_x"] = x
    fx["in_y"] = y.reshape(15, -1)
    fx["in_metric"] = np.float64(l2norm2_metric(y))

    # ---- entry-wise batch norm dataset (the reference pins only gradients on it); the
    # stored expectation is the training-mode definition in float64: per-entry mean and
    # Bessel-corrected variance over the mini-batch (the first 14 samples, as the test's
    # mini-batch size is num_samples // 2, and all 29), eps 1e-5, no scale or bias.
    np.random.seed(20190815)
    x = np.random.normal(size=(29, 7 * 5 * 3)).astype(np.float32)
    fx["ebn_x"] = x
    for tag, batch in (("mb14", x[:14]), ("all29", x)):
        xd = batch.astype(np.float64)
        mean = xd.mean(axis=0)
        var = xd.var(axis=0, ddof=1)
        fx[f"ebn_{tag}_mean"] = mean
        fx[f"ebn_{tag}_var"] = var
        fx[f"ebn_{tag}_y"] = (xd - mean) / np.sqrt(var + 1e-5)

    # ---- cross entropy dataset: 23 samples of (2*3, 64) U(0.25, 1) plus 64 labels in {0,1,2}.
    # The reference feeds channels 0..2 as the prediction, channels 3..5 as a dense ground
    # truth, and the labels as the ground truth of the use_labels cases; its metric is the
    # mean over samples of (1e-3 * loss)^2.
    np.random.seed(202303102)
    samples = np.random.uniform(low=0.25, high=1, size=(23, 6, 64)).astype(np.float32)
    labels = np.random.randint(3, size=(23, 1, 64)).astype(np.float32)
    pred, dense = samples[:, :3, :].reshape(23, 192), samples[:, 3:, :].reshape(23, 192)
    fx["ce_prediction"], fx["ce_dense_truth"], fx["ce_labels"] = pred, dense, labels.reshape(23, 64)
    pd = pred.astype(np.float64)
    loss_dense = -np.sum(dense.astype(np.float64) * np.log(pd), axis=1)
    lab = labels.reshape(23, 64).astype(np.int64)
    picked = np.take_along_axis(pd.reshape(23, 3, 64), lab[:, None, :], axis=1)[:, 0, :]
    loss_labels = -np.sum(np.log(picked), axis=1)
    fx["ce_loss_dense"], fx["ce_loss_labels"] = loss_dense, loss_labels
    fx["ce_metric_dense"] = np.float64(np.mean((1e-3 * loss_dense) ** 2))
    fx["ce_metric_labels"] = np.float64(np.mean((1e-3 * loss_labels) ** 2))
    fx["ce_metric_tol"] = np.float64(8 * np.finfo(np.float32).eps)  # relative, as in the reference

    # ---- entry-wise scale/bias: 29 x (7,5,3) N(0,1); scale N(1,1), bias N(0,1) per entry
    np.random.seed(20190723)
    x = np.random.normal(size=(29, 105)).astype(np.float32)
    scale = np.random.normal(loc=1, size=(7, 5, 3)).astype(np.float32)
    bias = np.random.normal(loc=0, size=(7, 5, 3)).astype(np.float32)
    y = scale.reshape(1, 105).astype(np.float64) * x.astype(np.float64) + bias.reshape(1, 105).astype(np.float64)
    fx["esb_x"], fx["esb_scale"], fx["esb_bias"], fx["esb_y"] = x, scale.reshape(105), bias.reshape(105), y
    fx["esb_metric"] = np.float64(l2norm2_metric(y))

    # ---- channel-wise scale/bias: 23 x (7,5,3) N(0,1); scale N(1,1), bias N(0,1) per channel
    np.random.seed(20190719)
    x = np.random.normal(size=(23, 105)).astype(np.float32)
    scale = np.random.normal(loc=1, size=(7, 1, 1)).astype(np.float32)
    bias = np.random.normal(loc=0, size=(7, 1, 1)).astype(np.float32)
    y = (scale.astype(np.float64) * x.reshape(23, 7, 5, 3).astype(np.float64) + bias.astype(np.float64)).reshape(23, 105)
    fx["csb_x"], fx["csb_scale"], fx["csb_bias"], fx["csb_y"] = x, scale.reshape(7), bias.reshape(7), y
    fx["csb_metric"] = np.float64(l2norm2_metric(y))

    np.savez_compressed(OUT, **fx)
    print(OUT, os.path.getsize(OUT), "bytes,", len(fx), "arrays")


if __name__ == "__main__":
    main()
