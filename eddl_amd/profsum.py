"""Turns rocprofv3's CSV output for a bench.py run into the short text tables kept under profiles/.

    python3 -m eddl_amd.profsum trace    <workload> <trace dir> <bench log> <out.txt>
    python3 -m eddl_amd.profsum traffic  <workload> <trace dir> <fetch dir> <write dir> <bench log> <out.txt> [<out.json>]
    python3 -m eddl_amd.profsum mfma     <workload> <counter dir> <out.txt>
    python3 -m eddl_amd.profsum stalls   <workload> <SQ counter dir> <TCP counter dir> <out.txt>
    python3 -m eddl_amd.profsum counters <title> <counter dir> <out.txt> [<kernel substring> ...]

Every table states in its header the rocprofv3 command that wrote the CSV files and the formula of each column.
The directories are those given to rocprofv3 with -d; the files in them are found by suffix
(*_kernel_stats.csv, *_kernel_trace.csv, *_counter_collection.csv), whatever host-name folder rocprofv3 put them in.
"""
import collections
import csv
import glob
import json
import os
import subprocess
import sys

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
COPY_PROBE_KIB = 262144.0  # bench.py --copy-probe: one ReLU over 2^26 floats reads 256 MiB and writes 256 MiB
HOT = ("conv_", "wino_", "maxpool", "avgpool", "dense", "bn_", "add_kernel", "concat", "scale_", "unary_kernel", "pad_", "softmax", "upsample")


def find(directory, suffix):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not hits:
        raise SystemExit("no *%s under %s" % (suffix, directory))
    return hits[0]


def rows(path):
    with open(path, newline="") as fh:
        return list(csv.DictReader(fh))


def counter(directory, name):
    """{kernel name: [value per dispatch]} of one counter; the per-dispatch value is the sum over the rows rocprofv3
    writes for it (one per XCD or shader engine, depending on the counter)."""
    per = collections.defaultdict(lambda: collections.defaultdict(float))
    for r in rows(find(directory, "_counter_collection.csv")):
        if r["Counter_Name"] == name:
            per[r["Kernel_Name"]][r["Dispatch_Id"]] += float(r["Counter_Value"])
    return {k: list(v.values()) for k, v in per.items()}


def durations(directory):
    """{kernel name: [End_Timestamp - Start_Timestamp in us per dispatch]} of a kernel trace."""
    d = collections.defaultdict(list)
    for r in rows(find(directory, "_kernel_trace.csv")):
        d[r["Kernel_Name"]].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return d


def bench_line(path):
    line = None
    for text in open(path, errors="replace"):
        if text.startswith('{"metric"'):
            line = json.loads(text)
    return line


def commit():
    """The commit the measured tree was built from: EDDLHIP_COMMIT if set (a copy of the tree without its .git), else git's HEAD."""
    if os.environ.get("EDDLHIP_COMMIT"):
        return os.environ["EDDLHIP_COMMIT"]
    try:
        here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        return subprocess.run(["git", "-C", here, "rev-parse", "--short", "HEAD"], capture_output=True, text=True, timeout=10).stdout.strip() or None
    except Exception:
        return None


def short(name, width):
    return name.replace("void (anonymous namespace)::", "").replace("(anonymous namespace)::", "")[:width]


def mean(values):
    return sum(values) / len(values)


def write(path, lines, workload=""):
    lines = [l.replace("WLTOKEN", workload) for l in lines]
    with open(path, "w") as fh:
        fh.write("\n".join(lines) + "\n")
    print("\n".join(lines))


def trace(workload, trace_dir, log, out, extra=""):
    stats = rows(find(trace_dir, "_kernel_stats.csv"))
    bench = bench_line(log)
    o = ["rocprofv3 kernel trace of the %s benchmark (MI355X, gfx950)%s" % (workload, ("; library at commit %s" % commit()) if commit() else ""),
         "commands (from the repository root):",
         "  rocprofv3 --kernel-trace --stats --output-format csv -d %s -o %s -- python3 bench.py --workload %s --steps 10 --warmup 3 --no-cpu-baseline --no-device-probe --no-workloads --no-dropin --plans gpurun_out/plans_WLTOKEN.txt%s > %s"
         % (trace_dir, workload, workload, extra, log),
         "  python3 -m eddl_amd.profsum trace %s %s %s %s" % (workload, trace_dir, log, out),
         "",
         "columns: rocprofv3's own *_kernel_stats.csv, unchanged: Name, Calls, TotalDurationNs, AverageNs (= TotalDurationNs / Calls),",
         "Percentage (= TotalDurationNs / sum of TotalDurationNs over all kernels x 100).  The run holds 3 warm-up + 10 timed steps and",
         "the repetitions bench.py uses to time the dominant kernel with HIP events.  The plans file comes from an earlier, unprofiled run",
         "of the same workload (python3 bench.py --workload W --steps 3 --warmup 1 --no-cpu-baseline --no-device-probe --no-workloads --no-dropin",
         "--plans gpurun_out/plans_W.txt), which searched the launch plans and saved what it found: the profiled run loads them and",
         "launches no search, so the trace holds the workload only, under the plans a default bench.py run uses.",
         "",
         "%-100s %6s %14s %12s %7s" % ("kernel", "calls", "total ns", "average ns", "%")]
    for r in stats:
        o.append("%-100s %6s %14s %12.0f %7.2f" % (short(r["Name"], 100), r["Calls"], r["TotalDurationNs"], float(r["AverageNs"]), float(r["Percentage"])))
    if bench:
        rf = bench["roofline"]
        o += ["", "bench.py line of the same run:",
              "  value %.1f %s, %.3f ms/step" % (bench["value"], bench["unit"], bench["ms_per_step"]),
              "  roofline kernel %s: %s launches/step, avg launch %.4f ms (HIP events inside bench.py), achieved %.2f %s = %.1f%% of %.1f"
              % (rf["kernel"], rf.get("launches_per_step"), rf.get("avg_launch_ms", 0.0), rf["achieved"], rf["unit"], 100 * rf["frac"], rf["peak"])]
        key = rf["kernel"].replace(" ", "")
        # (the trace spells out a kernel's defaulted last template argument, the library's name for it does not)
        dom = [r for r in stats if key in r["Name"].replace(" ", "").replace(",false>", ">")]
        if dom:
            o.append("  same kernel in the trace above: average %.4f ms over %s calls" % (float(dom[0]["AverageNs"]) / 1e6, dom[0]["Calls"]))
    write(out, o, workload)


def traffic(workload, trace_dir, fetch_dir, write_dir, log, out, out_json=None, extra=""):
    stats = rows(find(trace_dir, "_kernel_stats.csv"))
    f, w = counter(fetch_dir, "FETCH_SIZE"), counter(write_dir, "WRITE_SIZE")
    probe = [k for k in f if "unary_kernel<0>" in k]
    if not probe:
        raise SystemExit("the counter runs hold no copy probe: run bench.py with --copy-probe")
    sf, sw = COPY_PROBE_KIB / max(f[probe[0]]), COPY_PROBE_KIB / max(w[probe[0]])
    bench = bench_line(log)
    args = "--workload %s%s --steps 2 --warmup 1 --no-cpu-baseline --no-device-probe --no-workloads --no-dropin --plans gpurun_out/plans_WLTOKEN.txt --copy-probe" % (workload, extra)
    o = ["HBM traffic per launch of the %s benchmark kernels%s (MI355X, gfx950)%s"
         % (workload, " run layer by layer" if "--unfused" in extra else "", ("; library at commit %s" % commit()) if commit() else ""),
         "commands (from the repository root; one counter per run):",
         "  rocprofv3 --pmc FETCH_SIZE --output-format csv -d %s -o f -- python3 bench.py %s" % (fetch_dir, args),
         "  rocprofv3 --pmc WRITE_SIZE --output-format csv -d %s -o w -- python3 bench.py %s" % (write_dir, args),
         "  python3 -m eddl_amd.profsum traffic %s %s %s %s %s %s" % (workload, trace_dir, fetch_dir, write_dir, log, out),
         "  (%s is the directory of the kernel trace of the same workload, %s the output of that run)" % (trace_dir, log),
         "",
         "scale: --copy-probe adds one ReLU over 2^26 floats to the run (it reads 262144 KiB and writes 262144 KiB by construction);",
         "       FETCH_SIZE read %.1f KiB for it -> factor %.4f; WRITE_SIZE read %.1f KiB -> factor %.4f" % (max(f[probe[0]]), sf, max(w[probe[0]]), sw),
         "",
         "columns: calls = dispatches of the kernel in the counter run; FETCH / WRITE KiB avg = Counter_Value summed over the rows of one",
         "dispatch, averaged over the kernel's dispatches (launches of one kernel differ in size from layer to layer);",
         "HBM bytes/launch = (FETCH avg x fetch factor + WRITE avg x write factor) x 1024; avg us = AverageNs / 1000 of the kernel in",
         "the kernel trace (*_kernel_stats.csv); GB/s = HBM bytes/launch / avg us / 1000; % = GB/s / 8000 (HBM peak 8 TB/s) x 100.",
         "",
         "%-92s %6s %14s %14s %16s %9s %8s %6s" % ("kernel", "calls", "FETCH KiB avg", "WRITE KiB avg", "HBM bytes/launch", "avg us", "GB/s", "%")]
    dur = {r["Name"]: float(r["AverageNs"]) / 1e3 for r in stats}
    per_kernel = {}
    for r in stats:
        k = r["Name"]
        if k not in f or k not in w or not any(t in k for t in HOT):
            continue
        fl, wl = list(f[k]), list(w[k])
        if "unary_kernel<0>" in k:  # the probe launch is not one of the workload's
            fl.remove(max(fl))
            wl.remove(max(wl))
            if not fl:
                continue
        fm, wm = mean(fl), mean(wl)
        b = (fm * sf + wm * sw) * 1024
        us = dur[k]
        o.append("%-92s %6d %14.1f %14.1f %16.4g %9.1f %8.0f %6.1f" % (short(k, 92), len(fl), fm, wm, b, us, b / us / 1e3, b / us / 1e3 / HBM_PEAK_GBS * 100))
        per_kernel[k] = (b, len(fl), fm * sf * 1024, wm * sw * 1024)
    if bench:
        o += ["", "bench.py line of the traced run: %.1f %s, %.3f ms/step" % (bench["value"], bench["unit"], bench["ms_per_step"])]
    write(out, o, workload)
    if out_json:
        # every kernel of the table by name (as bench.py spells it: no blanks, no "void (anonymous namespace)::" prefix, no
        # parameter list), so that a later run finds its dominant kernel whichever plan its search kept
        table = {}
        for k, (b, calls, fb, wb) in per_kernel.items():
            name = short(k, 10 ** 6).split("(")[0].replace(" ", "")
            table[name] = {"hbm_bytes_per_launch": b, "fetch_bytes_per_launch": fb, "write_bytes_per_launch": wb, "launches_in_counter_run": calls}
        # forwards in the counter run (warm-up, timed steps, bench.py's per-op timing passes): the dominant kernel's dispatches
        # over its launches per forward
        steps = None
        if bench and bench["roofline"].get("launches_per_step"):
            dom = bench["roofline"]["kernel"].replace(" ", "")
            hit = [v for k, v in table.items() if k.replace(",false>", ">") == dom]
            if hit:
                steps = hit[0]["launches_in_counter_run"] / bench["roofline"]["launches_per_step"]
        with open(out_json, "w") as fh:
            json.dump({"kernels": table, "fetch_scale": sf, "write_scale": sw, "steps_in_counter_run": steps,
                       "dominant_kernel_of_that_run": bench["roofline"]["kernel"] if bench else None,
                       "launches_per_step_of_it": bench["roofline"].get("launches_per_step") if bench else None, "source": out, "commit": commit()}, fh, indent=1)
            fh.write("\n")


MFMA_COUNTERS = "SQ_INSTS_VALU_MFMA_MOPS_F32 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES GRBM_GUI_ACTIVE"


def mfma(workload, directory, out):
    mops, busy, gui = counter(directory, "SQ_INSTS_VALU_MFMA_MOPS_F32"), counter(directory, "SQ_VALU_MFMA_BUSY_CYCLES"), counter(directory, "GRBM_GUI_ACTIVE")
    dur = durations(directory)
    o = ["Matrix-core counters of the %s benchmark kernels (MI355X, gfx950)%s" % (workload, ("; library at commit %s" % commit()) if commit() else ""),
         "commands (from the repository root):",
         "  rocprofv3 --pmc %s --kernel-trace --output-format csv -d %s -o m -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu-baseline --no-workloads --no-dropin --plans gpurun_out/plans_WLTOKEN.txt"
         % (MFMA_COUNTERS, directory, workload),
         "  python3 -m eddl_amd.profsum mfma %s %s %s" % (workload, directory, out),
         ""]
    probe = [k for k in mops if "mfma_f32_probe" in k]
    if probe:
        m = mean(mops[probe[0]])
        o += ["SQ_INSTS_VALU_MFMA_MOPS_F32 counts fp32 matrix operations in units of 512 flops: the pure-MFMA probe kernel of the same run",
              "(mfma_f32_probe_kernel, 1.0737e12 flops per launch by construction) reads %.4g, i.e. %.1f flops per count." % (m, 1.0737e12 / m)]
    o += ["columns: calls = dispatches; avg us = mean of End_Timestamp - Start_Timestamp in THIS run (kernels run a few % slower while",
          "counters are collected); exec GFLOP = mean SQ_INSTS_VALU_MFMA_MOPS_F32 per dispatch x 512 / 1e9 (includes the zero taps of a",
          "padded K range); TFLOP/s = exec GFLOP / avg us / 1000; %peak = TFLOP/s / 157.3 x 100; busy % = SQ_VALU_MFMA_BUSY_CYCLES /",
          "(GRBM_GUI_ACTIVE / 8 XCDs x 1024 SIMDs) x 100; GHz = GRBM_GUI_ACTIVE / 8 / avg us / 1000 (the shader clock the kernel ran at:",
          "the 157.3 TFLOP/s peak is 256 CUs x 256 flops/clock x 2.4 GHz).",
          "",
          "%-88s %6s %9s %12s %9s %7s %7s %6s" % ("kernel", "calls", "avg us", "exec GFLOP", "TFLOP/s", "%peak", "busy %", "GHz")]
    for k in mops:
        if not any(t in k for t in ("conv_tap", "conv_gen", "conv_pointwise", "wino_fused_kernel", "dense_partial", "mfma_f32_probe")):
            continue
        us = mean(dur[k])
        fl = mean(mops[k]) * 512.0
        cyc = mean(gui[k]) / 8.0
        o.append("%-88s %6d %9.1f %12.2f %9.1f %7.1f %7.1f %6.2f"
                 % (short(k, 88), len(dur[k]), us, fl / 1e9, fl / us / 1e6, fl / us / 1e6 / FP32_MFMA_PEAK_TFLOPS * 100, 100 * mean(busy[k]) / (cyc * 1024.0), cyc / us / 1e3))
    write(out, o, workload)


STALL_SQ = "SQ_WAVES SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_WAIT_INST_ANY SQ_VALU_MFMA_BUSY_CYCLES SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_WAIT_INST_LDS GRBM_GUI_ACTIVE"
STALL_TCP = "SQ_INSTS_VALU SQ_INSTS_LDS SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_ANY SQ_WAIT_ANY TCP_PENDING_STALL_CYCLES_sum GRBM_GUI_ACTIVE"


def stalls(workload, sq_dir, tcp_dir, out):
    """Where the wavefronts of the convolution kernels spend their cycles: two counter passes over one bench.py run."""
    a = {n: counter(sq_dir, n) for n in STALL_SQ.split()}
    b = {n: counter(tcp_dir, n) for n in STALL_TCP.split()}
    dur = durations(sq_dir)
    o = ["Wavefront stall counters of the %s benchmark's convolution kernels (MI355X, gfx950)%s" % (workload, ("; library at commit %s" % commit()) if commit() else ""),
         "commands (from the repository root; two passes, the hardware holds 8 SQ counters at a time):",
         "  rocprofv3 --pmc %s --kernel-trace --output-format csv -d %s -o m -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu-baseline --no-device-probe --no-workloads --no-dropin --plans gpurun_out/plans_WLTOKEN.txt" % (STALL_SQ, sq_dir, workload),
         "  rocprofv3 --pmc %s --kernel-trace --output-format csv -d %s -o m -- python3 bench.py --workload %s --steps 2 --warmup 1 --no-cpu-baseline --no-device-probe --no-workloads --no-dropin --plans gpurun_out/plans_WLTOKEN.txt" % (STALL_TCP, tcp_dir, workload),
         "  python3 -m eddl_amd.profsum stalls %s %s %s %s" % (workload, sq_dir, tcp_dir, out),
         "",
         "columns (each counter: Counter_Value of a dispatch, averaged over the kernel's dispatches; SQ counters are sampled on one of the",
         "eight XCDs' shader engines and ratios of two of them are therefore scale-free):",
         "  avg us     mean End_Timestamp - Start_Timestamp in the first pass",
         "  mfma busy  SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 x 1024 SIMDs) x 100: share of SIMD-cycles with the matrix pipe busy",
         "  wait any   SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES x 100: share of its resident cycles a wavefront waits on s_waitcnt (memory or LDS)",
         "  wait lds   SQ_WAIT_INST_LDS / SQ_WAVE_CYCLES x 100",
         "  issue      SQ_ACTIVE_INST_ANY / SQ_WAVE_CYCLES x 100 (second pass): share of resident cycles a wavefront issues an instruction",
         "  tcp stall  TCP_PENDING_STALL_CYCLES_sum / (GRBM_GUI_ACTIVE / 8 x 256 CUs) x 100 (second pass): share of CU-cycles the vector",
         "             L1 holds requests back behind pending ones",
         "  valu/vmem  SQ_INSTS_VALU / (SQ_INSTS_VMEM_RD + SQ_INSTS_VMEM_WR): vector ALU instructions per vector memory instruction",
         "",
         "%-64s %6s %9s %10s %9s %9s %7s %10s %10s" % ("kernel", "calls", "avg us", "mfma busy", "wait any", "wait lds", "issue", "tcp stall", "valu/vmem")]
    for k in a["SQ_WAVE_CYCLES"]:
        if not ("conv_" in k or "wino_fused_kernel" in k) or k not in b["SQ_WAVE_CYCLES" if "SQ_WAVE_CYCLES" in b else "SQ_WAIT_ANY"]:
            continue
        m = lambda d, n: mean(d[n][k])
        cyc_a, cyc_b = m(a, "GRBM_GUI_ACTIVE") / 8.0, m(b, "GRBM_GUI_ACTIVE") / 8.0
        wc = m(a, "SQ_WAVE_CYCLES")
        # second-pass ratios use that pass's own wave cycles, estimated from the first pass scaled by the cycle counts
        wc_b = wc * cyc_b / cyc_a
        o.append("%-64s %6d %9.1f %10.1f %9.1f %9.1f %7.1f %10.1f %10.1f"
                 % (short(k, 64), len(dur[k]), mean(dur[k]), 100 * m(a, "SQ_VALU_MFMA_BUSY_CYCLES") / (cyc_a * 1024),
                    100 * m(a, "SQ_WAIT_INST_ANY") / wc, 100 * m(a, "SQ_WAIT_INST_LDS") / wc, 100 * m(b, "SQ_ACTIVE_INST_ANY") / wc_b,
                    100 * m(b, "TCP_PENDING_STALL_CYCLES_sum") / (cyc_b * 256), m(b, "SQ_INSTS_VALU") / (m(b, "SQ_INSTS_VMEM_RD") + m(b, "SQ_INSTS_VMEM_WR"))))
    write(out, o, workload)


def counters(title, directory, out, wanted):
    """A plain table of whatever counters a run collected: one row per kernel, mean per dispatch."""
    names, table = [], collections.defaultdict(dict)
    for r in rows(find(directory, "_counter_collection.csv")):
        if r["Counter_Name"] not in names:
            names.append(r["Counter_Name"])
    for n in names:
        for k, v in counter(directory, n).items():
            table[k][n] = (mean(v), len(v))
    o = [title, "source: %s; values are Counter_Value summed over the rows of one dispatch, averaged over the kernel's dispatches" % find(directory, "_counter_collection.csv"), "",
         "%-72s %6s " % ("kernel", "calls") + " ".join("%26s" % n[:26] for n in names)]
    for k, v in table.items():
        if wanted and not any(t in k for t in wanted):
            continue
        o.append("%-72s %6d " % (short(k, 72), max(c for _, c in v.values())) + " ".join("%26.5g" % v.get(n, (float("nan"), 0))[0] for n in names))
    write(out, o)


def main(argv):
    if len(argv) < 2:
        raise SystemExit(__doc__)
    cmd, a = argv[1], argv[2:]
    extra = ""
    if "--unfused" in a:
        a.remove("--unfused")
        extra = " --unfused"
    if cmd == "trace":
        trace(a[0], a[1], a[2], a[3], extra)
    elif cmd == "traffic":
        traffic(a[0], a[1], a[2], a[3], a[4], a[5], a[6] if len(a) > 6 else None, extra)
    elif cmd == "mfma":
        mfma(a[0], a[1], a[2])
    elif cmd == "stalls":
        stalls(a[0], a[1], a[2], a[3])
    elif cmd == "counters":
        counters(a[0], a[1], a[2], a[3:])
    else:
        raise SystemExit(__doc__)


if __name__ == "__main__":
    main(sys.argv)
