"""Times forward and backward of every layer of the library over shapes that the benchmark
configurations do not touch: rows off the 16-byte grid, rows just past a power of two, a few
channels or columns, very wide mini-batches, 16-bit storage.  One line per case with the
fraction of the 8 TB/s HBM peak on algorithmic bytes (forward 2 tensors, backward 3); cases
under --threshold percent in either direction are marked `<<<`.  The sweep exists to find
paths that leave most of the device idle (a helper kernel with a handful of workgroups, one
thread per row, ...), which no single benchmark shape would show.

    python -m lbann_amd.shape_sweep [--threshold 30] [--only SUBSTR] [--steps 8]

Needs a GPU; timings are event-bracketed loops on the current stream with resident tensors.
"""
import argparse

import numpy as np
import torch

from lbann_amd import layers as L

F, H = torch.float32, torch.float16


def _time(fwd, bwd, steps):
    for _ in range(2):
        fwd()
        bwd()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    ev[0].record()
    for _ in range(steps):
        fwd()
    ev[1].record()
    for _ in range(steps):
        bwd()
    ev[2].record()
    torch.cuda.synchronize()
    return ev[0].elapsed_time(ev[1]) / steps * 1e3, ev[1].elapsed_time(ev[2]) / steps * 1e3


def _mats(h, w, dt=F, positive=False):
    x = L.DeviceMatrix(h, w, dtype=dt)
    x.tensor.normal_()
    if positive:
        x.tensor.abs_().add_(0.05)
    dy = L.DeviceMatrix(h, w, dtype=dt)
    dy.tensor.normal_()
    return x, dy


def _tag(dt):
    return "f16" if dt == H else "f32"


def cases():
    """Yields (name, bytes of one tensor, forward callable, backward callable, tensors read+written fwd, bwd)."""
    # softmax family: odd lengths, lengths just past powers of two, few long rows, 16-bit storage
    for dt in (F, H):
        for h, w in [(257, 65536), (513, 32768), (1001, 16384), (1025, 16384), (2049, 8192), (4097, 4096),
                     (8193, 2048), (30522, 2048), (50257, 1024), (128256, 256), (21, 1 << 20), (1000003, 16)]:
            if dt == H:
                w //= 2 if h * w * 2 > (128 << 20) else 1
            for kind in ("softmax", "log_softmax"):
                layer = L.softmax_layer() if kind == "softmax" else L.log_softmax_layer()
                x, dy = _mats(h, w, dt)
                yield (f"{kind} {_tag(dt)} {h}x{w}", x.tensor.element_size() * h * w,
                       (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    for dims, w in [((64, 1001), 256), ((12, 197, 197), 32), ((1000, 49), 512), ((8, 100003), 32)]:
        layer = L.channelwise_softmax_layer(dims)
        h = int(np.prod(dims))
        x, dy = _mats(h, w)
        yield (f"channelwise_softmax f32 dims={dims} w={w}", 4 * h * w,
               (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    # layer norm: odd lengths with and without weights, both storage types
    for dt in (F, H):
        for n, w in [(257, 65536), (1001, 16384), (1025, 16384), (4099, 4096), (10001, 2048), (12290, 1024), (50001, 512)]:
            for weights in (False, True):
                layer = L.layer_norm_layer((n,), scale=weights, bias=weights)
                x, dy = _mats(n, w, dt)
                yield (f"layer_norm {_tag(dt)} n={n} w={w} weights={weights}", x.tensor.element_size() * n * w,
                       (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    for dims, w in [((3, 299, 299), 64), ((256, 7, 7), 1024), ((64, 13, 13), 512), ((1024, 1), 8192)]:
        layer = L.instance_norm_layer(dims)
        h = int(np.prod(dims))
        x, dy = _mats(h, w)
        yield (f"instance_norm f32 dims={dims} w={w}", 4 * h * w,
               (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    # batch norm: odd feature maps, a few channels, outside training, 16-bit storage
    for dt in (F, H):
        for dims, w, training in [((96, 55, 55), 64, True), ((64, 111, 111), 32, True), ((2048, 7, 7), 256, True),
                                  ((3, 299, 299), 64, True), ((3, 300, 300), 64, True), ((16384, 1), 512, True),
                                  ((256, 56, 56), 64, False), ((16, 150, 150), 32, False)]:
            layer = L.batch_normalization_layer(dims)
            h = int(np.prod(dims))
            x, dy = _mats(h, w, dt)
            layer.forward(x)
            layer.training = training
            yield (f"batch_norm {_tag(dt)} dims={dims} w={w} training={training}", x.tensor.element_size() * h * w,
                   (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    # entry-wise batch norm: odd heights, few rows under a wide mini-batch, outside training
    for h, w, training in [(100003, 128, True), (4096, 2048, True), (512, 4096, True), (16384, 512, True),
                           (100352, 512, True), (4096, 2048, False)]:
        layer = L.entrywise_batch_normalization_layer((h,))
        x, dy = _mats(h, w)
        layer.forward(x)
        layer.training = training
        yield (f"entrywise_batch_norm f32 {h}x{w} training={training}", 4 * h * w,
               (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3 if training else 2)
    # the layers either side
    for dt in (F, H):
        for h, w in [(1001, 16384), (21, 1 << 20), (50257, 256), (10, 262144)]:
            layer = L.cross_entropy_layer((h,))
            x, t = _mats(h, w, dt, positive=True)
            t.tensor.abs_()
            dl = L.DeviceMatrix(1, w, dtype=dt)
            dl.tensor.normal_()
            yield (f"cross_entropy {_tag(dt)} {h}x{w}", x.tensor.element_size() * h * w,
                   (lambda l=layer, a=x, b=t: l.forward(a, b)), (lambda l=layer, g=dl: l.backward(g)), 2, 4)
    for classes, spatial, w in [(21, 512 * 512, 8), (19, 1024 * 2048, 1), (1000, 1, 65536)]:
        layer = L.cross_entropy_layer((classes, spatial), use_labels=True)
        h = classes * spatial
        x, _ = _mats(h, w, positive=True)
        t = L.DeviceMatrix(spatial, w)
        t.tensor.random_(0, classes)
        dl = L.DeviceMatrix(1, w)
        dl.tensor.normal_()
        yield (f"cross_entropy labels classes={classes} spatial={spatial} w={w}", 4 * h * w,
               (lambda l=layer, a=x, b=t: l.forward(a, b)), (lambda l=layer, g=dl: l.backward(g)), 1, 1)
    for dims, w in [((96, 55, 55), 64), ((3, 299, 299), 64), ((4096, 1, 1), 4096)]:
        layer = L.channelwise_scale_bias_layer(dims)
        h = int(np.prod(dims))
        x, dy = _mats(h, w)
        yield (f"channelwise_scale_bias f32 dims={dims} w={w}", 4 * h * w,
               (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)
    for h, w in [(100003, 128), (4096, 2048)]:
        layer = L.entrywise_scale_bias_layer((h,))
        x, dy = _mats(h, w)
        yield (f"entrywise_scale_bias f32 {h}x{w}", 4 * h * w,
               (lambda l=layer, a=x: l.forward(a)), (lambda l=layer, g=dy: l.backward(g)), 2, 3)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--threshold", type=float, default=30.0, help="percent of 8 TB/s under which a case is marked")
    ap.add_argument("--only", default="", help="run the cases whose name contains this")
    ap.add_argument("--steps", type=int, default=8)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("shape_sweep needs a GPU")
    L.capi.lib()
    slow = 0
    print("| case | fwd us | % of 8 TB/s | bwd us | % of 8 TB/s | |")
    print("|---|---|---|---|---|---|")
    for name, nbytes, fwd, bwd, nf, nb in cases():
        if args.only not in name:
            continue
        tf, tb = _time(fwd, bwd, args.steps)
        pf, pb = nf * nbytes / tf / 8e4, nb * nbytes / tb / 8e4
        mark = "<<<" if min(pf, pb) < args.threshold else ""
        slow += bool(mark)
        print(f"| {name} | {tf:.1f} | {pf:.1f} | {tb:.1f} | {pb:.1f} | {mark} |", flush=True)
    print(f"\n{slow} case(s) under {args.threshold:g} % of the HBM peak in one direction or the other.")


if __name__ == "__main__":
    main()
