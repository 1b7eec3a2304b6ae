"""Times single convolution layers of libeddlhip.so back to back, outside any network.

    python3 -m eddl_amd.convbench layers  <shapes file | resnet50 | vgg16> [--reps R]
    python3 -m eddl_amd.convbench planfit <shapes file | resnet50 | vgg16> [--reps R]
    python3 -m eddl_amd.convbench one     N C H W Kf R S stride pad [flags] [--tile T --slices S] [--reps R]
    python3 -m eddl_amd.convbench timeline N C H W Kf R S stride pad [flags] [--tile T --slices S]

A shape line reads  N C H W Kf R S stride pad count [flags];  flags: b = inference BatchNorm in the epilogue, r = ReLU,
s = residual add.  `count` is how often the layer occurs in the network (weights the totals).

layers   one row per layer: time per launch, TFLOP/s = 2 N Kf C R S P Q / time, % of the 157.3 TFLOP/s fp32 MFMA peak,
         GB/s = 4 (N C H W + Kf C R S + N Kf P Q [x2 with a residual]) / time, and the kernel the planner launched.
planfit  the planner's choice against every (tile family, K slices) plan forced through eddlhip_conv2d_force_plan: how far
         the planned launch is from the fastest forced one, per layer and summed over the list.
one      a single layer, optionally with a forced plan.
timeline one launch of a single layer (1x1, 2x2 or 3x3 filters) with eddlhip_conv2d_trace switched on: every workgroup
         leaves four stamps of the device's 100 MHz clock (entry, first operands in LDS, end of the K loop, stores
         drained) and the CU it ran on.  Printed: how long the three phases last per workgroup (shader cycles at the
         engine clock the records themselves give), how many workgroups a CU holds and how many of them are inside their
         K loop at a time (share of the launch), and the timeline of one CU.  A workgroup outside its K loop uses no
         matrix instruction: the second histogram is the supply side of the matrix pipe.

Launches repeat back to back on one stream between two events, so the figures include no host gaps; a layer timed this
way runs somewhat slower than inside a network (the same launch forty times in a row keeps the chip at its power limit
and finds nothing of its input in the last-level cache), which is why network figures come from kernel traces of
bench.py instead.  This tool is for comparing plans and kernels with each other.
"""
import argparse
import time

import numpy as np

import eddl_amd

PEAK_TFLOPS = 157.3

RESNET50 = """
64 3 224 224 64 7 7 2 3 1 br
64 64 56 56 256 1 1 1 0 1 b
64 64 56 56 64 1 1 1 0 1 br
64 64 56 56 64 3 3 1 1 3 br
64 64 56 56 256 1 1 1 0 3 brs
64 256 56 56 64 1 1 1 0 2 br
64 256 56 56 512 1 1 2 0 1 b
64 256 56 56 128 1 1 1 0 1 br
64 128 56 56 128 3 3 2 1 1 br
64 128 28 28 512 1 1 1 0 4 brs
64 512 28 28 128 1 1 1 0 3 br
64 128 28 28 128 3 3 1 1 3 br
64 512 28 28 1024 1 1 2 0 1 b
64 512 28 28 256 1 1 1 0 1 br
64 256 28 28 256 3 3 2 1 1 br
64 256 14 14 1024 1 1 1 0 6 brs
64 1024 14 14 256 1 1 1 0 5 br
64 256 14 14 256 3 3 1 1 5 br
64 1024 14 14 2048 1 1 2 0 1 b
64 1024 14 14 512 1 1 1 0 1 br
64 512 14 14 512 3 3 2 1 1 br
64 512 7 7 2048 1 1 1 0 3 brs
64 2048 7 7 512 1 1 1 0 2 br
64 512 7 7 512 3 3 1 1 2 br
"""

VGG16 = """
32 3 224 224 64 3 3 1 1 1 r
32 64 224 224 64 3 3 1 1 1 r
32 64 112 112 128 3 3 1 1 1 r
32 128 112 112 128 3 3 1 1 1 r
32 128 56 56 256 3 3 1 1 1 r
32 256 56 56 256 3 3 1 1 2 r
32 256 28 28 512 3 3 1 1 1 r
32 512 28 28 512 3 3 1 1 2 r
32 512 14 14 512 3 3 1 1 3 r
"""

TILE_FAMILIES = 4
SLICES = (1, 2, 3, 4, 6, 8, 12, 16)


def shapes(source):
    text = {"resnet50": RESNET50, "vgg16": VGG16}.get(source) or open(source).read()
    out = []
    for line in text.strip().splitlines():
        f = line.split()
        if not f or f[0].startswith("#"):
            continue
        out.append(([int(v) for v in f[:9]], int(f[9]) if len(f) > 9 else 1, f[10] if len(f) > 10 else ""))
    return out


def warm(hip, seconds=0.15):
    a, b = hip.full((1 << 24,), 1.0), hip.empty((1 << 24,))
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        hip.relu(a, b)
        hip.synchronize()


class Layer:
    def __init__(self, hip, dims, flags, rng):
        N, C, H, W, Kf, R, S, st, pad = dims
        self.hip, self.dims, self.flags = hip, dims, flags
        self.P, self.Q = (H + 2 * pad - R) // st + 1, (W + 2 * pad - S) // st + 1
        self.x = hip.array(rng.standard_normal((N, C, H, W), dtype=np.float32))
        self.w = hip.array((rng.standard_normal((Kf, C, R, S)) * 0.05).astype(np.float32))
        self.out = hip.empty((N, Kf, self.P, self.Q))
        self.bn = (hip.full((Kf,), 1.0), hip.full((Kf,), 0.1), hip.full((Kf,), 0.0), hip.full((Kf,), 1.0), 1e-5) if "b" in flags else None
        self.res = hip.array(rng.standard_normal((N, Kf, self.P, self.Q), dtype=np.float32)) if "s" in flags else None
        hip.cache_conv_filters(self.w)
        self.flops = 2.0 * N * Kf * C * R * S * self.P * self.Q
        self.bytes = 4.0 * (N * C * H * W + Kf * C * R * S + N * Kf * self.P * self.Q * (2 if self.res is not None else 1))

    def call(self):
        st, pad = self.dims[7], self.dims[8]
        self.hip.conv2D(self.x, self.w, None, self.out, st, st, pad, pad, bn=self.bn, residual=self.res, relu="r" in self.flags)

    def time_us(self, reps, warm_seconds=0.03):
        # the same launch for a few tens of milliseconds first: after the idle time that building the tensors leaves,
        # the clocks need that long to settle, and a measurement that starts earlier favours whatever runs later
        t0 = time.perf_counter()
        while True:
            for _ in range(3):
                self.call()
            self.hip.synchronize()
            if time.perf_counter() - t0 >= warm_seconds:
                break
        s, e = self.hip.event(), self.hip.event()
        s.record()
        for _ in range(reps):
            self.call()
        e.record()
        self.hip.synchronize()
        return s.elapsed_ms(e) * 1e3 / reps

    def close(self):
        self.hip.uncache_conv_filters(self.w)


def row(layer, us, count):
    d = " ".join(str(v) for v in layer.dims) + " " + layer.flags
    tf = layer.flops / us / 1e6
    return "%-36s x%d %8.1f us %7.1f TFLOP/s %5.1f%%  %6.0f GB/s  %s" % (d, count, us, tf, tf / PEAK_TFLOPS * 100, layer.bytes / us / 1e3, layer.hip.last_conv_kernel())


def cmd_layers(hip, source, reps):
    rng = np.random.default_rng(0)
    tot_us = tot_fl = 0.0
    for dims, count, flags in shapes(source):
        layer = Layer(hip, dims, flags, rng)
        us = layer.time_us(reps)
        print(row(layer, us, count), flush=True)
        tot_us += us * count
        tot_fl += layer.flops * count
        layer.close()
    print("TOTAL %.1f us  %.1f TFLOP/s (%.1f%% of %.1f)" % (tot_us, tot_fl / tot_us / 1e6, tot_fl / tot_us / 1e6 / PEAK_TFLOPS * 100, PEAK_TFLOPS))


def cmd_planfit(hip, source, reps):
    rng = np.random.default_rng(0)
    tot_auto = tot_best = 0.0
    for dims, count, flags in shapes(source):
        layer = Layer(hip, dims, flags, rng)
        hip.force_conv_plan(-1, 1)
        auto = layer.time_us(reps)
        kernel = hip.last_conv_kernel()
        best, best_plan = auto, "planned"
        for tile in range(TILE_FAMILIES):
            for slices in SLICES:
                hip.force_conv_plan(tile, slices)
                try:
                    us = layer.time_us(reps)
                except eddl_amd.EddlHipError:
                    continue  # the plan does not apply to this layer (more slices than K steps, ...)
                if us < best:
                    best, best_plan = us, "tile %d x %d slices" % (tile, slices)
        hip.force_conv_plan(-1, 1)
        d = " ".join(str(v) for v in dims) + " " + flags
        print("%-36s x%d planned %8.1f us (%s)  fastest %8.1f us (%s)  planned/fastest %.3f" % (d, count, auto, kernel, best, best_plan, auto / best), flush=True)
        tot_auto += auto * count
        tot_best += best * count
        layer.close()
    print("SUM planned %.1f us  fastest forced %.1f us  ratio %.3f" % (tot_auto, tot_best, tot_auto / tot_best))


def cmd_timeline(hip, dims, flags, tile, slices):
    layer = Layer(hip, dims, flags, np.random.default_rng(0))
    hip.force_conv_plan(tile, slices)
    us = layer.time_us(20, warm_seconds=0.2)
    buf = hip.conv_trace(1 << 16)
    try:
        for _ in range(3):
            layer.call()
        hip.synchronize()
    finally:
        hip.conv_trace(0)
        hip.force_conv_plan(-1, 1)
    rec = buf.numpy().view(np.uint64).reshape(-1, 8)
    rec = rec[rec[:, 0] != 0].astype(np.int64)
    n = len(rec)
    print("%s %s  %s  %.1f us per launch untraced, %d workgroups" % (" ".join(str(v) for v in dims), flags, hip.last_conv_kernel(), us, n))
    if n == 0:
        print("no records: the launch was not one of the traced kernels")
        return
    t = rec[:, 0:4] - rec[:, 0].min()
    mhz = float(np.median((rec[:, 6] - rec[:, 5]) / np.maximum(t[:, 3] - t[:, 0], 1))) * 100.0
    t = (t * (mhz / 100.0)).astype(np.int64)  # shader cycles
    span = int(t[:, 3].max())
    print("engine clock %.0f MHz (shader-clock difference over 100 MHz-clock difference, median over the workgroups); the launch "
          "spans %d cycles = %.1f us with the stores drained" % (mhz, span, span / mhz))
    phases = (("entry -> first operands in LDS", t[:, 1] - t[:, 0]), ("K loop", t[:, 2] - t[:, 1]), ("K loop end -> stores drained", t[:, 3] - t[:, 2]),
              ("workgroup lifetime", t[:, 3] - t[:, 0]))
    for name, v in phases:
        print("  %-30s mean %7.0f  median %7.0f  p10 %7.0f  p90 %7.0f cycles  (mean %.2f us)" % (name, v.mean(), np.median(v), np.percentile(v, 10), np.percentile(v, 90), v.mean() / mhz))
    cu = ((rec[:, 4] >> 8) & 0xff) | (((rec[:, 4] >> 32) & 0xf) << 8)  # CU, shader array and engine bits of HW_ID, XCC_ID above them
    cus = np.unique(cu)
    in_loop, resident = np.zeros(10), np.zeros(10)
    per_cu = []
    for c in cus:
        tt = t[cu == c]
        per_cu.append(len(tt))
        ev = sorted([(r[0], 0, 1) for r in tt] + [(r[1], 1, 0) for r in tt] + [(r[2], -1, 0) for r in tt] + [(r[3], 0, -1) for r in tt])
        a = b = last = 0
        for when, da, db in ev:
            in_loop[min(a, 9)] += when - last
            resident[min(b, 9)] += when - last
            a, b, last = a + da, b + db, when
        in_loop[0] += span - last
        resident[0] += span - last
    print("%d CUs; workgroups per CU %.2f (min %d, max %d)" % (len(cus), np.mean(per_cu), min(per_cu), max(per_cu)))
    print("share of the launch (%) by the number of a CU's workgroups that are     0     1     2     3     4     5     6     7     8    9+")
    print("  resident                                                         " + " ".join("%5.1f" % v for v in resident / resident.sum() * 100))
    print("  inside their K loop                                              " + " ".join("%5.1f" % v for v in in_loop / in_loop.sum() * 100))
    c0 = cus[len(cus) // 2]
    sel = np.where(cu == c0)[0]
    sel = sel[np.argsort(t[sel, 0])]
    print("one CU, thousands of cycles:   entry  K loop from      to  drained")
    for i in sel:
        print("                             %7.1f %12.1f %7.1f %8.1f" % tuple(t[i] / 1e3))
    layer.close()


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("cmd", choices=["layers", "planfit", "one", "timeline"])
    ap.add_argument("args", nargs="+")
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--tile", type=int, default=-1)
    ap.add_argument("--slices", type=int, default=1)
    a = ap.parse_args()
    hip = eddl_amd.Backend(0)
    warm(hip)
    if a.cmd == "layers":
        cmd_layers(hip, a.args[0], a.reps)
    elif a.cmd == "planfit":
        cmd_planfit(hip, a.args[0], a.reps)
    elif a.cmd == "timeline":
        cmd_timeline(hip, [int(v) for v in a.args[:9]], a.args[9] if len(a.args) > 9 else "", a.tile, a.slices)
    else:
        dims = [int(v) for v in a.args[:9]]
        flags = a.args[9] if len(a.args) > 9 else ""
        layer = Layer(hip, dims, flags, np.random.default_rng(0))
        hip.force_conv_plan(a.tile, a.slices)
        print(row(layer, layer.time_us(a.reps), 1))
        hip.force_conv_plan(-1, 1)
        layer.close()


if __name__ == "__main__":
    main()
