"""Synthetic inputs of the benchmark configurations (host arrays, seeded).

All matrices are (height, width) NumPy arrays in Fortran order, one column per
sample.  The generator is numpy.random.default_rng(0x4C420000 + cfg), so the CPU
baseline, the parity tests and the GPU benchmark see identical values.
"""
import numpy as np


def _rng(cfg):
    return np.random.default_rng(0x4C420000 + cfg)


def _normal(rng, h, w, mean=0.0, std=1.0):
    a = rng.standard_normal((w, h), dtype=np.float32)
    if std != 1.0:
        a *= np.float32(std)
    if mean != 0.0:
        a += np.float32(mean)
    return a.T  # Fortran-ordered (h, w) view


def cfg1_layer_norm(h=1024, w=128):
    """LayerNorm fp32, 1024 features x 128 samples, eps 1e-5, scale 1, bias 0."""
    rng = _rng(1)
    return dict(x=_normal(rng, h, w), dy=_normal(rng, h, w), eps=1e-5,
                scale=np.ones(h, np.float32), bias=np.zeros(h, np.float32), dims=(h,))


def cfg2_softmax(h=32768, w=512):
    """Softmax / LogSoftmax fp32: logits N(0, 2^2), 1% of entries set to +30."""
    rng = _rng(2)
    x = _normal(rng, h, w, 0.0, 2.0)
    mask = rng.random((w, h), dtype=np.float32).T < np.float32(0.01)
    x = np.where(mask, np.float32(30.0), x)
    x = np.asfortranarray(x)
    return dict(x=x, dy=_normal(rng, h, w))


def cfg3_batch_norm(N=64, C=256, H=56, W=56):
    """BatchNorm training fp32, NCHW 64x256x56x56 stored as (C*H*W) x N."""
    rng = _rng(3)
    h = C * H * W
    return dict(x=_normal(rng, h, N, 2.0, 3.0), dy=_normal(rng, h, N), eps=1e-5, decay=0.9,
                scale=rng.uniform(0.5, 1.5, C).astype(np.float32),
                bias=(0.1 * rng.standard_normal(C)).astype(np.float32), dims=(C, H, W))


def cfg4_layer_norm_f16(h=4096, w=8192):
    """LayerNorm fp16 storage: column j ~ N(mu_j, sigma_j^2), mu_j ~ U(-50, 50),
    sigma_j ~ LogU(1e-3, 1e2); values are rounded to fp16 before anyone sees them."""
    rng = _rng(4)
    mu = rng.uniform(-50.0, 50.0, w).astype(np.float32)
    sigma = np.exp(rng.uniform(np.log(1e-3), np.log(1e2), w)).astype(np.float32)
    x = rng.standard_normal((w, h), dtype=np.float32)
    x *= sigma[:, None]
    x += mu[:, None]
    x = x.astype(np.float16).T
    dy = rng.standard_normal((w, h), dtype=np.float32).astype(np.float16).T
    return dict(x=x, dy=dy, eps=1e-5,
                scale=(1.0 + 0.1 * rng.standard_normal(h)).astype(np.float32),
                bias=(0.1 * rng.standard_normal(h)).astype(np.float32), dims=(h,))


def cfg5a_channelwise_softmax(C=64, S=4096, w=256):
    """ChannelwiseSoftmax fp32, 256 samples x 64 channels x 4096 spatial."""
    rng = _rng(5)
    h = C * S
    return dict(x=_normal(rng, h, w), dy=_normal(rng, h, w), dims=(C, S))


def cfg5b_wide_softmax(h=262144, w=16):
    """Softmax fp32 over 262144 classes x 16 samples (split reduction per column)."""
    rng = _rng(6)
    return dict(x=_normal(rng, h, w), dy=_normal(rng, h, w))


def extra_entrywise_batch_norm(h=1048576, w=64):
    """Entry-wise batch norm fp32 (not a baseline configuration): 2^20 entries x 64 samples."""
    rng = _rng(7)
    return dict(x=_normal(rng, h, w, 2.0, 3.0), dy=_normal(rng, h, w), eps=1e-5, decay=0.9, dims=(h,))


# algorithmic (compulsory) bytes: forward reads x and writes y, backward reads two
# tensors and writes one; per-column / per-channel vectors are not counted.
def algorithmic_bytes(elements, elem_size):
    fwd = 2 * elements * elem_size
    bwd = 3 * elements * elem_size
    return fwd, bwd
