#!/usr/bin/env python3
"""Benchmark of the CNN forward path on one MI355X.

A step is one forward pass of the workload over one batch of synthetic input that is already
resident in HBM (default workload: VGG-16, batch 32, fp32, 3x224x224 - the configuration the
headline metric is quoted on).  Prints ONE JSON line on stdout; the per-layer table goes to
stderr with --layers and to DIR/bench_layers_<workload>.{json,txt} with --out DIR.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vgg16|block|resnet50|unet|conv]
                    [--no-cpu-baseline] [--layers] [--out DIR] [--unfused] [--graph]

--unfused runs the graph layer by layer (every BatchNorm, ReLU, Add and Pad as a launch of its own, as
the reference walks it): not the headline figure, but the run whose per-op table gives the HBM rate of
each bandwidth kernel at the workload's real tensor sizes.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix peak (256 CUs x 256 flop/clk x 2.4 GHz)
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name -> (builder kwargs, seed, input distribution, description)
    "vgg16": (dict(batch=32), 3, "uniform", "VGG-16 forward, batch 32, 3x224x224, fp32 (13 conv3x3+ReLU, 5 maxpool, 3 dense, softmax)"),
    "conv": (dict(batch=8), 1, "normal", "single Conv2D 3->32, 3x3 same, bias, batch 8, 3x32x32, fp32 (14 MFLOP: bound by launch latency)"),
    "block": (dict(batch=64), 2, "normal", "Conv3x3(64->64)-BN-ReLU-MaxPool2x2 block, batch 64, 64x56x56, fp32"),
    "resnet50": (dict(batch=64), 4, "normal", "ResNet-50 forward, batch 64, 3x224x224, fp32, inference BN"),
    "unet": (dict(batch=4), 5, "uniform", "U-Net forward, batch 4, 1x512x512, fp32"),
}


def builder_of(name):
    from eddl_amd import models
    return {"vgg16": models.vgg16, "block": models.conv_bn_relu_pool_block, "resnet50": models.resnet50, "unet": models.unet,
            "conv": models.single_conv}[name]


def build_workload(name):
    from eddl_amd import models
    kwargs, seed, dist, desc = WORKLOADS[name]
    builder = builder_of(name)
    model = builder(**kwargs)
    models.init_he_normal(model, seed)
    x = models.synthetic_input(model.lin[0].out_shape, seed + 1000, dist)
    return model, x, desc


def time_ops(hip, model, reps):
    """Per-op device time (ms, mean over reps) from events on the stream the kernels run on: the
    whole op (repack + kernels) between two events and, for convolutions, the launches of the
    convolution kernel alone, each bracketed inside the library."""
    n = len(model.ops)
    ev = [[(hip.event(), hip.event()) for _ in range(n)] for _ in range(reps)]
    kernels = [None] * n
    kern_ms = [0.0] * n
    kern_launches = [0] * n
    for r in range(reps):
        for i, op in enumerate(model.ops):
            s, e = ev[r][i]
            if op.kind == "conv2d":
                hip.conv_profile(True)
                s.record()
                op.run()
                e.record()
                launches, ms = hip.conv_profile_read()
                hip.conv_profile(False)
                kernels[i] = hip.last_conv_kernel().split(" +ksplit")[0]
                kern_ms[i] += ms / reps
                kern_launches[i] = launches
            else:
                s.record()
                op.run()
                e.record()
    hip.synchronize()
    op_ms = [float(np.mean([ev[r][i][0].elapsed_ms(ev[r][i][1]) for r in range(reps)])) for i in range(n)]
    return op_ms, kernels, kern_ms, kern_launches


PARITY_BOUND = 1e-4  # largest |device - oracle| over the sample's outputs, relative to the largest |oracle| output


def cpu_baseline(workload, want_seconds=20.0, device_output=None):
    """The CPU oracle (a port of the reference's CPU algorithm: per-image im2col + one
    single-threaded GEMM, OpenMP over the batch, separate bias/ReLU/pool passes) timed on this
    host on a bounded sample of the same workload.  The sample is the first images of the
    benchmark's own batch (same seeds), so with ``device_output`` (the device's output for the
    whole batch) the oracle's outputs also check the timed device run end to end: ``parity``."""
    from eddl_amd import models
    from oracle import net_oracle
    from oracle.oracle import Oracle
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    env_threads = os.environ.get("OMP_NUM_THREADS")
    if env_threads:
        cores = min(cores, int(env_threads))
    kwargs, seed, dist, _ = WORKLOADS[workload]
    builder = builder_of(workload)
    full_batch = kwargs["batch"]
    sample_batch = min(full_batch, max(1, cores))  # one image per thread: the reference parallelises over the batch
    result = {"unit": "images/sec", "cores": cores, "kind": "port"}
    for label, hpc in (("hpc", True), ("strict", False)):
        try:
            ora = Oracle(hpc=hpc)
        except (RuntimeError, OSError) as exc:
            result["value_" + label] = None
            result["note_" + label] = str(exc)
            continue
        ora.set_num_threads(cores)
        model = builder(**dict(kwargs, batch=sample_batch))
        models.init_he_normal(model, seed)
        # the first images of the benchmark's own batch: the stream is drawn row-major, so a smaller batch is its prefix
        # (a normal fill draws values in pairs, and every image of the configurations holds an even number of values)
        x = models.synthetic_input(model.lin[0].out_shape, seed + 1000, dist)
        budget = want_seconds * (0.6 if hpc else 0.4)
        times = []
        while not times or (sum(times) < budget and len(times) < 200):
            t0 = time.perf_counter()
            ref = net_oracle.forward(ora, model, [x], conv_algo="im2col")[0]
            times.append(time.perf_counter() - t0)
        if not hpc and device_output is not None:  # the strict build is the parity oracle
            got = np.asarray(device_output)[:sample_batch].reshape(ref.shape)
            scale = float(np.abs(ref).max())
            err = float(np.abs(got - ref).max())
            result["parity"] = {"images": sample_batch, "max_abs_err": err, "max_abs_ref": scale,
                                "err_over_max_ref": err / scale if scale > 0 else err, "bound": PARITY_BOUND,
                                "ok": bool(err <= PARITY_BOUND * scale)}
        # the first forward pays for page faults of the lowered-matrix buffers: drop it when there are others
        timed = times[1:] if len(times) > 1 else times
        dt = sum(timed) / len(timed)
        result["value_" + label] = sample_batch / dt
        result["seconds_" + label] = sum(times)
        result["forwards_" + label] = len(times)
    result["value"] = result.get("value_hpc") or result.get("value_strict")
    result["sample"] = ("repeated forwards of the same model on a batch of %d (of %d), same seeds, about 20 s of CPU work in all "
                        "(forwards_*/seconds_* give the counts; mean of all but the first); im2col + single-threaded GEMM per image, "
                        "OpenMP over the batch, %d threads; value = -O3 -march=x86-64-v3 -ffast-math build (the reference's HPC "
                        "flags), value_strict = -O2 without FMA contraction (the parity oracle)" % (sample_batch, full_batch, cores))
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="vgg16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--layers", action="store_true", help="print the per-op table to stderr")
    ap.add_argument("--out", default=None, metavar="DIR", help="also write the per-op table and the result into this directory")
    ap.add_argument("--unfused", action="store_true",
                    help="one launch per layer (no Conv+BN+Add+ReLU / Pad / Dense+ReLU fusion): measures the stand-alone bandwidth kernels")
    ap.add_argument("--graph", action="store_true",
                    help="record the plan once as a graph and replay it with one call per step (for plans of short kernels)")
    ap.add_argument("--conv-algo", default="auto", choices=["auto", "mfma_staged", "mfma_lds"], help="input gather of the convolution kernels")
    ap.add_argument("--no-device-probe", action="store_true",
                    help="skip the pure-MFMA probe of the device's sustained fp32 matrix rate (keeps kernel traces to the workload)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="after the timed region run one ReLU over 2^26 floats (reads 256 MiB, writes 256 MiB): the plain copy "
                         "kernel of known size that scales FETCH_SIZE / WRITE_SIZE counter readings")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on ONE GPU (the forward path has no collectives); --gpus %d is not supported" % args.gpus)

    import eddl_amd
    hip = eddl_amd.Backend(0)
    hip.set_conv_algo(args.conv_algo)
    model, x, desc = build_workload(args.workload)
    model.build(hip, fuse=not args.unfused)
    batch = x.shape[0]
    model.input_tensor().copy_from(x)  # input resident in HBM before the timed region
    hip.synchronize()

    step = model.run
    if args.graph:
        model.capture()
        step = model.run_graph
    for _ in range(args.warmup):
        step()
    hip.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    hip.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    out_host = model.out[id(model.lout[0])].numpy()
    if not np.all(np.isfinite(out_host)):
        sys.exit("bench.py: non-finite output")

    if args.copy_probe:
        probe_in, probe_out = hip.full((1 << 26,), 1.0), hip.empty((1 << 26,))
        hip.relu(probe_in, probe_out)
        hip.synchronize()
        del probe_in, probe_out

    # ---- per-op device times (events on the kernels' stream), same resident input
    reps = max(3, min(args.steps, 10))
    op_ms, op_kernels, kern_ms, kern_launches = time_ops(hip, model, reps)
    # what an event pair reads around a kernel that does next to nothing (one float filled): the part of every
    # per-op figure below that is not the op
    tiny = hip.empty((1,))
    pairs = [(hip.event(), hip.event()) for _ in range(50)]
    for s, e in pairs:
        s.record()
        hip.fill_(tiny, 0.0)
        e.record()
    hip.synchronize()
    event_floor_ms = float(np.median([s.elapsed_ms(e) for s, e in pairs]))
    rows = []
    for op, ms, kern, kms, kl in zip(model.ops, op_ms, op_kernels, kern_ms, kern_launches):
        row = {"op": op.kind, "name": op.name, "ms": ms, "flops": op.flops, "bytes": op.bytes}
        if kern:
            row.update(kernel=kern, kernel_ms=kms, kernel_launches=kl)
        if op.kind in ("conv2d", "dense") and ms > 0:
            row["tflops"] = op.flops / ms / 1e9
            row["frac_fp32_mfma_peak"] = row["tflops"] / PEAK_FP32_MFMA_TFLOPS
        if ms > 0:
            row["gbs"] = op.bytes / ms / 1e6
            row["frac_hbm_peak"] = row["gbs"] / PEAK_HBM_GBS
        rows.append(row)

    # ---- dominant kernel: the convolution kernel (one template instance = one symbol in a
    # rocprofv3 kernel trace) that accounts for the most device time in a step
    conv_rows = [r for r in rows if r["op"] == "conv2d"]
    by_kernel = {}
    for r in conv_rows:
        by_kernel.setdefault(r.get("kernel", "?"), []).append(r)
    dom_name, dom = max(by_kernel.items(), key=lambda kv: sum(r["kernel_ms"] for r in kv[1]))
    dom_flops, dom_ms = sum(r["flops"] for r in dom), sum(r["kernel_ms"] for r in dom)
    dom_launches = sum(r["kernel_launches"] for r in dom)
    achieved = dom_flops / dom_ms / 1e9 if dom_ms > 0 else 0.0
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic_%s.json" % args.workload)
    if os.path.exists(tpath) and not args.unfused:  # the committed counter runs are of the fused plan
        with open(tpath) as fh:
            traffic = json.load(fh).get("hbm_bytes_per_launch")
    roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_FP32_MFMA_TFLOPS, "traffic": traffic,
                "kernel": dom_name, "launches_per_step": dom_launches, "layers": len(dom),
                "flops_per_launch": dom_flops / max(dom_launches, 1), "avg_launch_ms": dom_ms / max(dom_launches, 1),
                "algorithmic_bytes_per_launch": sum(r["bytes"] for r in dom) / max(dom_launches, 1)}

    # what the matrix pipe sustains on this device with nothing else running (constant operands, then
    # operands that change every instruction): the published peak assumes the top clock throughout
    if not args.no_device_probe:
        const_mean, const_best, _ = hip.probe_mfma_f32(vary_operands=False, launches=30)
        vary_mean, vary_best, vary_worst = hip.probe_mfma_f32(vary_operands=True, launches=60)
        roofline["device_probe"] = {"unit": "TFLOP/s", "pure_mfma_constant_operands": const_mean,
                                    "pure_mfma_varying_operands_mean": vary_mean, "varying_best_launch": vary_best,
                                    "varying_worst_launch": vary_worst,
                                    "frac_of_varying_mean": achieved / vary_mean if vary_mean > 0 else None}
        # and what plain read / write / copy streams over 1 GiB buffers sustain, beside the 8 TB/s HBM peak
        rd, wr, cp = hip.probe_hbm(1 << 30)
        roofline["device_probe"].update(hbm_unit="GB/s", hbm_read_stream=rd, hbm_write_stream=wr, hbm_copy_stream=cp)

    conv_ms = sum(r["ms"] for r in conv_rows)
    conv_flops = sum(r["flops"] for r in conv_rows)
    result = {
        "metric": "%s forward images/sec (fp32, 1 GPU%s)" % (args.workload, ", layer by layer" if args.unfused else ""),
        "value": batch * args.steps / wall, "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded He-normal weights, U(0,1)/N(0,1) inputs, resident in HBM)",
        "config": {"workload": desc, "batch": batch, "fused": not args.unfused, "fused_ops": len(model.ops), "graph_replay": bool(args.graph), "device": hip.name},
        "roofline": roofline,
        "conv_total": {"tflops": conv_flops / conv_ms / 1e9 if conv_ms else 0.0, "ms": conv_ms, "gflop": conv_flops / 1e9,
                       "frac_fp32_mfma_peak": (conv_flops / conv_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS) if conv_ms else 0.0},
        "device_ms_sum_of_ops": sum(op_ms),
        "event_pair_floor_ms": event_floor_ms,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, device_output=out_host)
        parity = result["cpu_baseline"].get("parity")
        if parity is not None and not parity["ok"]:
            print(json.dumps(result))
            sys.exit("bench.py: the device's output differs from the CPU oracle's by %.3g of the largest output (bound %.0e)"
                     % (parity["err_over_max_ref"], PARITY_BOUND))

    table = ["# ms = device time between two events around the op; an event pair around a one-element fill reads %.4f ms"
             % event_floor_ms,
             "%-44s %9s %9s %8s %9s %7s" % ("op", "ms", "TFLOP/s", "%mfma", "GB/s", "%hbm")]
    for r in rows:
        table.append("%-44s %9.4f %9s %8s %9.1f %7.2f  %s" % (
            r["name"][:44], r["ms"], "%.2f" % r["tflops"] if "tflops" in r else "-",
            "%.1f" % (100 * r["frac_fp32_mfma_peak"]) if "tflops" in r else "-", r.get("gbs", 0.0), 100 * r.get("frac_hbm_peak", 0.0),
            r.get("kernel", "")))
    if args.layers:
        print("\n".join(table), file=sys.stderr)
    out_dir = args.out
    if out_dir:
        os.makedirs(out_dir, exist_ok=True)
        stem = "bench_layers_%s%s" % (args.workload, "_unfused" if args.unfused else "")
        with open(os.path.join(out_dir, stem + ".json"), "w") as fh:
            json.dump({"result": result, "ops": rows}, fh, indent=1)
        with open(os.path.join(out_dir, stem + ".txt"), "w") as fh:
            fh.write("\n".join(table) + "\n")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
