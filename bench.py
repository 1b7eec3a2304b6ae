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
                kernels[i] = hip.last_conv_kernel()
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


def oracle_parity(workload, device_output, max_images):
    """End-to-end check of a device output against the CPU oracle (strict build) on the first images of the
    workload's own batch; no timing.  The threads a small sample leaves idle share each image's convolutions
    (same arithmetic)."""
    from eddl_amd import models
    from oracle import net_oracle
    from oracle.oracle import Oracle
    kwargs, seed, dist, _ = WORKLOADS[workload]
    n = min(kwargs["batch"], max_images)
    ora = Oracle(hpc=False)
    ora.set_inner_parallel(True)
    try:
        model = builder_of(workload)(**dict(kwargs, batch=n))
        models.init_he_normal(model, seed)
        x = models.synthetic_input(model.lin[0].out_shape, seed + 1000, dist)
        ref = net_oracle.forward(ora, model, [x], conv_algo="im2col")[0]
    finally:
        ora.set_inner_parallel(False)
    got = np.asarray(device_output)[:n].reshape(ref.shape)
    scale, err = float(np.abs(ref).max()), float(np.abs(got - ref).max())
    return {"images": n, "max_abs_err": err, "max_abs_ref": scale, "err_over_max_ref": err / scale if scale > 0 else err,
            "bound": PARITY_BOUND, "ok": bool(err <= PARITY_BOUND * scale)}


RIDGE_FLOP_PER_BYTE = PEAK_FP32_MFMA_TFLOPS * 1e3 / PEAK_HBM_GBS  # 19.7: below it a layer is bound by HBM, not by the matrix cores


def measure(hip, workload, steps, warmup, fused=True, graph=False, tune=True, plans=None):
    """Builds the workload, runs `warmup` + `steps` forwards with the input resident in HBM, then times every op.
    Returns (summary dict, per-op rows, device output of the last forward, model description)."""
    model, x, desc = build_workload(workload)
    model.build(hip, fuse=fused)
    batch = x.shape[0]
    model.input_tensor().copy_from(x)  # input resident in HBM before the timed region
    hip.synchronize()
    if tune:
        # the library's plan search (the reference's cudnnFindConvolutionForwardAlgorithm on a layer's first forward): with the
        # clocks warm, one forward in which every new convolution geometry is run under every launch plan; all of it
        # before the timed region
        if plans and os.path.exists(plans):
            hip.conv_tuned_load(plans)   # what an earlier run found: nothing left to search for these geometries
            hip.conv_autotune(True)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.1:
            model.run()
            hip.synchronize()
        hip.conv_autotune(True)
        model.run()
        hip.synchronize()
        hip.workspace_trim()   # (the search has done so itself wherever its candidates grew the workspace)
        if plans:
            hip.conv_tuned_save(plans)
    plans_info = None
    if tune:
        # the table the run ended up with (sorted lines of eddlhip_conv2d_tuned_save): its hash names the plans this line was measured under
        import hashlib
        import tempfile
        with tempfile.NamedTemporaryFile("r", suffix=".txt") as fh:
            hip.conv_tuned_save(fh.name)
            lines = sorted(l.strip() for l in open(fh.name) if l.strip() and not l.startswith("#"))
        forms = {"planner": 0, "direct_tile": 0, "winograd_three_kernels": 0, "winograd_folded": 0, "winograd_one_launch": 0, "upsampled_2x2": 0}
        for l in lines:
            tile = int(l.split("|")[1].split()[0])
            forms["planner" if tile < 0 else "direct_tile" if tile < 4 else "winograd_three_kernels" if tile == 4 else "winograd_folded" if tile == 5
                  else "winograd_one_launch" if tile < 8 else "upsampled_2x2"] += 1
        plans_info = {"geometries": len(lines), "sha16": hashlib.sha256("\n".join(lines).encode()).hexdigest()[:16], "kept": forms,
                      "workspace_bytes_after_search": hip.workspace_bytes()}
    step = model.run
    if graph:
        model.capture()
        step = model.run_graph
    for _ in range(warmup):
        step()
    hip.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    hip.synchronize()
    wall = time.perf_counter() - t0
    out_host = model.out[id(model.lout[0])].numpy()
    if not np.all(np.isfinite(out_host)):
        sys.exit("bench.py: non-finite output (%s)" % workload)

    # ---- per-op device times (events on the kernels' stream), same resident input
    reps = max(3, min(steps, 10))
    op_ms, op_kernels, kern_ms, kern_launches = time_ops(hip, model, reps)
    rows = []
    for op, ms, kern, kms, kl in zip(model.ops, op_ms, op_kernels, kern_ms, kern_launches):
        row = {"op": op.kind, "name": op.name, "ms": ms, "flops": op.flops, "bytes": op.bytes}
        if kern:
            # kernel_flops: what the timed kernel itself multiplies.  The Winograd form times its product launch (16 products
            # of [Kf x C] by [C x blocks] matrices, 2.25 times fewer multiplications than the layer's direct count); the two
            # transform kernels around it are in the op's own time only
            kernel_flops, form = op.flops, "direct"
            if kern.startswith("winograd["):
                blocks = int(kern[kern.rindex(",") + 1:].split()[0])
                kern = kern[len("winograd["):kern.rindex(",")]
                conv = [l for l in op.layers if "cd" in l.attrs][0].attrs["cd"]
                n_out, kf = conv.out_shape[0] * conv.out_shape[2] * conv.out_shape[3], conv.out_shape[1]
                c_in = op.flops // (2 * conv.kr * conv.kc * n_out * kf)
                positions = (conv.kr + 1) * (conv.kc + 1)          # 16 products for a 3x3 filter, 9 for a 2x2 one
                kernel_flops, form = 2 * positions * kf * c_in * blocks, "winograd"
            elif kern.startswith("upsampled2x2["):
                # a 2x2 filter on an input upsampled twice, as four convolutions of the stored image: 9 products per channel
                # and stored pixel ("block") where the direct form has 16
                blocks = int(kern[kern.rindex(",") + 1:].split()[0])
                kern = kern[len("upsampled2x2["):kern.rindex(",")]
                conv = [l for l in op.layers if "cd" in l.attrs][0].attrs["cd"]
                n_out, kf = conv.out_shape[0] * conv.out_shape[2] * conv.out_shape[3], conv.out_shape[1]
                c_in = op.flops // (2 * conv.kr * conv.kc * n_out * kf)
                kernel_flops, form = 2 * 9 * kf * c_in * blocks, "upsampled2x2"
            row.update(kernel=kern.split(" +ksplit")[0], kernel_ms=kms, kernel_launches=kl, kernel_flops=kernel_flops, form=form)
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
    dom_flops, dom_ms = sum(r["kernel_flops"] for r in dom), sum(r["kernel_ms"] for r in dom)
    dom_launches = sum(r["kernel_launches"] for r in dom)
    achieved = dom_flops / dom_ms / 1e9 if dom_ms > 0 else 0.0
    roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_FP32_MFMA_TFLOPS, "traffic": None,
                "kernel": dom_name, "launches_per_step": dom_launches, "layers": len(dom),
                "flops_per_launch": dom_flops / max(dom_launches, 1), "avg_launch_ms": dom_ms / max(dom_launches, 1),
                "algorithmic_bytes_per_launch": sum(r["bytes"] for r in dom) / max(dom_launches, 1)}
    # HBM bytes per launch of that kernel come from committed counter runs (two rocprofv3 --pmc passes cannot run
    # inside this process); they are reported only when the file names the kernel this run found dominant
    tpath = os.path.join(ROOT, "profiles", "traffic_%s.json" % workload)
    if os.path.exists(tpath) and fused:  # the committed counter runs are of the fused plan; the file lists every kernel of them by name
        with open(tpath) as fh:
            t = json.load(fh)
        # (a kernel trace spells out a defaulted last template argument, the library's name for the kernel does not)
        table = {k.replace(",false>", ">"): v for k, v in t.get("kernels", {}).items()}
        entry = table.get(dom_name.replace(" ", ""))
        if entry:
            roofline["traffic"] = entry["hbm_bytes_per_launch"]
            roofline["traffic_fetch_bytes"], roofline["traffic_write_bytes"] = entry.get("fetch_bytes_per_launch"), entry.get("write_bytes_per_launch")
            roofline["traffic_measured_at_commit"] = t.get("commit")
            per_step = entry["launches_in_counter_run"] / max(t.get("steps_in_counter_run", 1), 1)
            if abs(per_step - dom_launches) > 1e-9:  # the plan search gave that kernel other layers in this run than in the counter runs
                roofline["traffic_note"] = ("profiles/traffic_%s.json averages %.4g launches per step of this kernel, this run has %d"
                                            % (workload, per_step, dom_launches))
        else:
            roofline["traffic_note"] = "profiles/traffic_%s.json has no row for this run's dominant kernel" % workload
    # convolutions whose arithmetic intensity is below the ridge (first layers with 1-3 input channels, 1-filter
    # last layers): priced against the HBM roof
    hbm_bound = [{"name": r["name"], "kernel": r.get("kernel"), "ms": r.get("kernel_ms", r["ms"]),
                  "flop_per_byte": r["flops"] / r["bytes"], "gbs": r["bytes"] / r.get("kernel_ms", r["ms"]) / 1e6,
                  "frac_hbm_peak": r["bytes"] / r.get("kernel_ms", r["ms"]) / 1e6 / PEAK_HBM_GBS}
                 for r in conv_rows if r["bytes"] > 0 and r["flops"] / r["bytes"] < RIDGE_FLOP_PER_BYTE and r.get("kernel_ms", r["ms"]) > 0]
    conv_ms = sum(r["ms"] for r in conv_rows)
    conv_flops = sum(r["flops"] for r in conv_rows)
    executed_flops = sum(r.get("kernel_flops", r["flops"]) for r in conv_rows)  # what the launches multiply (Winograd layers: 2.25x less)
    summary = {"value": batch * steps / wall, "unit": "images/sec", "ms_per_step": wall * 1e3 / steps, "steps": steps, "warmup": warmup,
               "batch": batch, "fused_ops": len(model.ops), "roofline": roofline, "hbm_bound_convs": hbm_bound,
               # the layers' direct-form flop count over their device time: layers that run in the Winograd form multiply 2.25
               # times less, so this is an effective rate and may pass the matrix peak; the roofline entry above prices the
               # dominant kernel by what it multiplies itself
               "conv_total": {"tflops": conv_flops / conv_ms / 1e9 if conv_ms else 0.0, "ms": conv_ms, "gflop": conv_flops / 1e9,
                              "frac_fp32_mfma_peak": (conv_flops / conv_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS) if conv_ms else 0.0,
                              "flops_counted": "direct form", "layers": len(conv_rows),
                              # the flops the launches really multiply over the same time: the matrix pipe's useful share
                              "executed_gflop": executed_flops / 1e9,
                              "mfma_util": (executed_flops / conv_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS) if conv_ms else 0.0,
                              "winograd_layers": sum(1 for r in conv_rows if r.get("form") == "winograd")},
               "device_ms_sum_of_ops": sum(op_ms), "plans": plans_info, "workspace_bytes": hip.workspace_bytes()}
    del model
    return summary, rows, out_host, desc


def dropin_path():
    """VGG-16, batch 32, through the drop-in route: the C++ host layer (the reference's Tensor / Layer / Net classes and
    eddl:: functions over the binding's gpu_* functions), each mode in a child process of its own that builds the net from
    the benchmark's seeds, lets the binding's gpu_init switch the plan search on (nothing in the environment) and times 20
    forwards with the input resident: `layer_walk` is what an unchanged EDDL program gets (one gpu_* call per layer, a wait
    after each, as the reference's wrappers wait), `fused_plan` the same net after eddl_hip::fuse(net)."""
    import subprocess
    import tempfile
    driver = os.path.join(ROOT, "eddl_amd", "host", "net_driver")
    if not os.path.exists(driver):
        return {"note": "eddl_amd/host/net_driver is not built"}
    result = {"workload": WORKLOADS["vgg16"][3], "unit": "images/sec", "plan_search": "on (gpu_init)", "host": "C++ (eddl_amd/host, tests/host/net_driver.cpp)"}
    env = {k: v for k, v in os.environ.items() if k not in ("EDDLHIP_NO_TUNE", "EDDLHIP_PLANS", "EDDLHIP_PLANS_SAVE")}
    with tempfile.TemporaryDirectory() as tmp:
        for key, flags in (("layer_walk", "time"), ("fused_plan", "fused+time")):
            cmd = [driver, flags + ":vgg16", "synth:3", "synth:1003:uniform", os.path.join(tmp, "y.raw"), "32", "224", "1000", "64", "128", "256", "512", "512", "4096"]
            try:
                res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300, env=env)
            except subprocess.TimeoutExpired:
                result[key] = {"note": "timed out"}
                continue
            line = [l for l in res.stdout.splitlines() if l.startswith("ms_per_forward")]
            if res.returncode != 0 or not line:
                result[key] = {"note": "net_driver failed: " + (res.stderr or res.stdout)[-300:]}
                continue
            f = line[0].split()
            result[key] = {"value": float(f[3]), "ms_per_forward": float(f[1]), "workspace_bytes": int(f[5]), "tuned_geometries": int(f[7])}
    return result


# the other configurations, run after the headline workload: (steps, warmup, images of the oracle's parity sample)
OTHER_WORKLOADS = {"conv": (200, 20, 8), "block": (50, 5, 16), "resnet50": (20, 5, 16), "unet": (10, 3, 2)}


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
    ap.add_argument("--no-workloads", action="store_true",
                    help="report the headline workload only (without it a default VGG-16 run also measures the other four "
                         "configurations, briefly, into the 'workloads' object of the JSON line)")
    ap.add_argument("--no-dropin", action="store_true",
                    help="skip the two child processes that time VGG-16 through the C++ host layer (the 'dropin' object of the JSON line)")
    ap.add_argument("--no-tune", action="store_true",
                    help="keep the launch planner's own choice for every convolution (without it the library searches the launch "
                         "plans of every convolution geometry once, before the timed region: eddlhip_conv2d_autotune)")
    ap.add_argument("--plans", default=None, metavar="FILE",
                    help="start the plan search from the plans in FILE (if it exists) and write what the run ends up with back to it: "
                         "a second run with the same file launches no search (kernel traces then hold the workload only)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="after the timed region run one ReLU over 2^26 floats (reads 256 MiB, writes 256 MiB): the plain copy "
                         "kernel of known size that scales FETCH_SIZE / WRITE_SIZE counter readings")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on ONE GPU (the forward path has no collectives); --gpus %d is not supported" % args.gpus)

    import eddl_amd
    hip = eddl_amd.Backend(0)
    hip.set_conv_algo(args.conv_algo)
    summary, rows, out_host, desc = measure(hip, args.workload, args.steps, args.warmup, fused=not args.unfused, graph=args.graph, tune=not args.no_tune, plans=args.plans)
    batch = summary["batch"]
    ms_per_step = summary["ms_per_step"]
    roofline = summary["roofline"]
    achieved = roofline["achieved"]

    if args.copy_probe:
        probe_in, probe_out = hip.full((1 << 26,), 1.0), hip.empty((1 << 26,))
        hip.relu(probe_in, probe_out)
        hip.synchronize()
        del probe_in, probe_out

    # what an event pair reads around a kernel that does next to nothing (one float filled): the part of every
    # per-op figure that is not the op
    tiny = hip.empty((1,))
    pairs = [(hip.event(), hip.event()) for _ in range(50)]
    for s, e in pairs:
        s.record()
        hip.fill_(tiny, 0.0)
        e.record()
    hip.synchronize()
    event_floor_ms = float(np.median([s.elapsed_ms(e) for s, e in pairs]))

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

    result = {
        "metric": "%s forward images/sec (fp32, 1 GPU%s)" % (args.workload, ", layer by layer" if args.unfused else ""),
        "value": summary["value"], "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (mt19937 + Box-Muller: He-normal weights from the configuration's seed, U(0,1)/N(0,1) inputs from seed + 1000; resident in HBM)",
        "config": {"workload": desc, "batch": batch, "fused": not args.unfused, "fused_ops": summary["fused_ops"], "graph_replay": bool(args.graph), "plan_search": not args.no_tune,
                   "device": hip.name},
        "roofline": roofline,
        "hbm_bound_convs": summary["hbm_bound_convs"],
        "conv_total": summary["conv_total"],
        "device_ms_sum_of_ops": summary["device_ms_sum_of_ops"],
        "plans": summary["plans"], "workspace_bytes": summary["workspace_bytes"],
        "event_pair_floor_ms": event_floor_ms,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, device_output=out_host)
        parity = result["cpu_baseline"].get("parity")
        if parity is not None and not parity["ok"]:
            print(json.dumps(result))
            sys.exit("bench.py: the device's output differs from the CPU oracle's by %.3g of the largest output (bound %.0e)"
                     % (parity["err_over_max_ref"], PARITY_BOUND))

    # ---- the other configurations, each for a fraction of a second of device time: throughput, dominant kernel against
    # its roof, and the end-to-end parity of the timed run against the CPU oracle
    if args.workload == "vgg16" and not (args.no_workloads or args.unfused or args.graph):
        result["workloads"] = {}
        for w, (steps, warmup, parity_images) in OTHER_WORKLOADS.items():
            sm, _, out_w, desc_w = measure(hip, w, steps, warmup, tune=not args.no_tune)
            entry = {"workload": desc_w, "value": sm["value"], "unit": "images/sec", "ms_per_step": sm["ms_per_step"], "steps": steps,
                     "warmup": warmup, "batch": sm["batch"], "dominant_kernel": sm["roofline"]["kernel"],
                     "frac": sm["roofline"]["frac"], "achieved_tflops": sm["roofline"]["achieved"],
                     "avg_launch_ms": sm["roofline"]["avg_launch_ms"], "launches_per_step": sm["roofline"]["launches_per_step"],
                     "conv_total": sm["conv_total"], "hbm_bound_convs": sm["hbm_bound_convs"], "plans": sm["plans"],
                     "workspace_bytes": sm["workspace_bytes"], "traffic": sm["roofline"].get("traffic")}
            if not args.no_cpu_baseline:
                entry["parity"] = oracle_parity(w, out_w, parity_images)
            result["workloads"][w] = entry
        bad = [w for w, e in result["workloads"].items() if "parity" in e and not e["parity"]["ok"]]
        if bad:
            print(json.dumps(result))
            sys.exit("bench.py: the device's output differs from the CPU oracle's beyond %.0e of the largest output in: %s"
                     % (PARITY_BOUND, ", ".join(bad)))

    if args.workload == "vgg16" and not (args.no_dropin or args.unfused or args.graph or args.no_tune):
        result["dropin"] = dropin_path()

    table = ["# ms = device time between two events around the op; an event pair around a one-element fill reads %.4f ms"
             % event_floor_ms,
             "# TFLOP/s = the layer's direct-form flop count over that time (a layer in the Winograd form multiplies 2.25 times less: "
             "its rate is an effective one)",
             "%-44s %9s %9s %8s %9s %7s" % ("op", "ms", "TFLOP/s", "%mfma", "GB/s", "%hbm")]
    for r in rows:
        table.append("%-44s %9.4f %9s %8s %9.1f %7.2f  %s" % (
            r["name"][:44], r["ms"], "%.2f" % r["tflops"] if "tflops" in r else "-",
            "%.1f" % (100 * r["frac_fp32_mfma_peak"]) if "tflops" in r else "-", r.get("gbs", 0.0), 100 * r.get("frac_hbm_peak", 0.0),
            ("winograd: " if r.get("form") == "winograd" else "upsampled 2x2: " if r.get("form") == "upsampled2x2" else "") + r.get("kernel", "")))
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
