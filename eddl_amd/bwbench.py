"""Times the stand-alone bandwidth kernels of libeddlhip.so at the tensor sizes of the benchmark networks.

    python3 -m eddl_amd.bwbench [--reps R] [relu add bn maxpool avgpool pad concat scale ...]

One row per (kernel, shape): microseconds per launch (R launches back to back between two events, after a few
milliseconds of the same launch), the algorithmic bytes the operation must move (every input read once, every output
written once - the MaxPool's two index tensors and the BatchNorm's `opa` copy included), and GB/s = bytes / time with
its share of the 8 TB/s HBM peak.  Tensors here are larger than the 256 MB last-level cache only for the biggest
shapes; the smaller ones partly run out of it, as they do inside a network.
"""
import argparse
import time

import numpy as np

import eddl_amd

HBM_PEAK_GBS = 8000.0

# (N, C, H, W) of activations that the layer-by-layer ResNet-50 (batch 64), VGG-16 (batch 32) and U-Net (batch 4, 512x512)
# plans hand to these kernels
ACTIVATIONS = [(64, 64, 112, 112), (64, 256, 56, 56), (64, 64, 56, 56), (64, 512, 28, 28), (64, 128, 28, 28), (64, 1024, 14, 14),
               (64, 2048, 7, 7), (32, 64, 224, 224), (32, 512, 14, 14), (4, 64, 512, 512), (4, 256, 128, 128)]


def timed(hip, call, reps):
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.01:
        call()
        hip.synchronize()
    s, e = hip.event(), hip.event()
    s.record()
    for _ in range(reps):
        call()
    e.record()
    hip.synchronize()
    return s.elapsed_ms(e) * 1e3 / reps


def report(name, shape, us, nbytes, note=""):
    gbs = nbytes / us / 1e3
    print("%-10s %-22s %9.1f us %12.0f bytes %7.0f GB/s %5.1f%%  %s" % (name, "x".join(str(d) for d in shape), us, nbytes, gbs, gbs / HBM_PEAK_GBS * 100, note), flush=True)


def pooled(h, k, s, p):
    return (h + 2 * p - k) // s + 1


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("which", nargs="*")
    ap.add_argument("--reps", type=int, default=20)
    a = ap.parse_args()
    want = lambda k: not a.which or k in a.which
    hip = eddl_amd.Backend(0)
    for shape in ACTIVATIONS:
        n = int(np.prod(shape))
        N, C, H, W = shape
        x = hip.full(shape, 1.5)
        y = hip.empty(shape)
        if want("relu"):
            report("relu", shape, timed(hip, lambda: hip.relu(x, y), a.reps), 8.0 * n)
        if want("add"):
            z = hip.full(shape, 0.5)
            report("add", shape, timed(hip, lambda: hip.add(1.0, x, 1.0, z, y), a.reps), 12.0 * n)
            del z
        if want("bn"):
            opa = hip.empty(shape)
            g, b, m, v, sd = hip.full((C,), 1.1), hip.full((C,), 0.1), hip.full((C,), 0.2), hip.full((C,), 0.9), hip.empty((C,))
            report("bn", shape, timed(hip, lambda: hip.batchnorm_inference(x, y, opa, m, v, g, b, sd, 1e-5), a.reps), 12.0 * n, "x -> y, opa")
            del opa
        if want("maxpool") and H % 2 == 0 and H >= 14:
            for k, s, p in ((2, 2, 0), (3, 2, 1)):
                P, Q = pooled(H, k, s, p), pooled(W, k, s, p)
                o, ix, iy = hip.empty((N, C, P, Q)), hip.empty((N, C, P, Q)), hip.empty((N, C, P, Q))
                report("maxpool", shape, timed(hip, lambda: hip.mpool2D(x, o, ix, iy, (k, k), (s, s), (p, p, p, p)), a.reps), 4.0 * n + 12.0 * N * C * P * Q,
                       "%dx%d stride %d pad %d -> values, indX, indY" % (k, k, s, p))
                del o, ix, iy
        if want("avgpool") and H == 7:
            o = hip.empty((N, C, 1, 1))
            report("avgpool", shape, timed(hip, lambda: hip.avgpool2D(x, o, (H, W), (1, 1), (0, 0, 0, 0)), a.reps), 4.0 * n + 4.0 * N * C, "global")
            del o
        if want("pad") and N == 4:
            o = hip.empty((N, C, H + 1, W + 1))
            report("pad", shape, timed(hip, lambda: hip.pad(x, o, (0, 1, 1, 0)), a.reps), 4.0 * n + 4.0 * N * C * (H + 1) * (W + 1), "(top, right, bottom, left) = (0, 1, 1, 0)")
            del o
        if want("concat") and N == 4:
            o = hip.empty((N, 2 * C, H, W))
            report("concat", shape, timed(hip, lambda: hip.concat(o, [x, y], 1), a.reps), 16.0 * n, "two tensors along the channels")
            del o
        if want("scale") and N == 4 and H <= 256:
            o = hip.empty((N, C, 2 * H, 2 * W))
            report("scale", shape, timed(hip, lambda: hip.scale(x, o, (2 * H, 2 * W)), a.reps), 4.0 * n + 16.0 * n, "nearest, x2")
            del o
        del x, y


if __name__ == "__main__":
    main()
