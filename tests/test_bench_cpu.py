"""bench.py pieces that need no GPU: the refusal of more than one GPU, the workload table (FLOP
counts of the five configurations against figures worked out by hand from their layer shapes), and
the CPU-baseline leg on a tiny sample."""
import json
import os
import subprocess
import sys

import numpy as np

from conftest import ROOT


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         text=True, timeout=120)
    assert res.returncode != 0 and "ONE GPU" in res.stderr and res.stdout.strip() == ""


def test_workload_flops_match_the_configurations():
    sys.path.insert(0, ROOT)
    import bench
    want = {"vgg16": 982.18e9, "resnet50": 523.15e9, "unet": 1745.1e9, "block": 14.797e9, "conv": 14155776.0}
    for name, (kwargs, seed, dist, desc) in bench.WORKLOADS.items():
        m = bench.builder_of(name)(**kwargs)
        flops = 0
        for l in m.layers:
            if l.kind == "conv2d":
                cd = l.attrs["cd"]
                N, Kf, P, Q = cd.out_shape
                flops += 2 * N * Kf * cd.kz * cd.kr * cd.kc * P * Q
        assert abs(flops - want[name]) / want[name] < 2e-3, (name, flops)


def test_cpu_baseline_leg_runs_on_a_small_sample(monkeypatch):
    sys.path.insert(0, ROOT)
    import bench
    monkeypatch.setitem(bench.WORKLOADS, "block", ({"batch": 2, "channels": 4, "size": 8, "filters": 4}, 2, "normal", "tiny block"))
    out = bench.cpu_baseline("block", want_seconds=0.2)
    assert out["kind"] == "port" and out["unit"] == "images/sec" and out["cores"] >= 1
    assert out["value"] > 0 and out["value_strict"] > 0 and "sample" in out
    json.dumps(out)


def test_cpu_baseline_leg_checks_a_device_output_against_the_oracle(monkeypatch):
    """The parity gate of the benchmark: an output equal to the oracle's passes, one that is off by 1e-3 of the
    output scale does not; a larger batch than the sample is compared on its first images."""
    sys.path.insert(0, ROOT)
    import bench
    from eddl_amd import models
    from oracle import net_oracle
    from oracle.oracle import Oracle
    kwargs = {"batch": 2, "channels": 4, "size": 8, "filters": 4}
    monkeypatch.setitem(bench.WORKLOADS, "block", (kwargs, 2, "normal", "tiny block"))
    monkeypatch.setattr(os, "cpu_count", lambda: 1)   # a sample of one image out of the batch of two
    monkeypatch.setattr(os, "sched_getaffinity", lambda pid: {0}, raising=False)
    model = models.conv_bn_relu_pool_block(**kwargs)
    models.init_he_normal(model, 2)
    x = models.synthetic_input(model.lin[0].out_shape, 1002, "normal")   # the benchmark's own input: seed + 1000
    full = net_oracle.forward(Oracle(hpc=False), model, [x])[0]
    good = bench.cpu_baseline("block", want_seconds=0.1, device_output=full)["parity"]
    assert good["ok"] and good["images"] == 1 and good["max_abs_err"] == 0.0
    bad = bench.cpu_baseline("block", want_seconds=0.1, device_output=full + 1e-3 * np.abs(full).max())["parity"]
    assert not bad["ok"] and bad["err_over_max_ref"] > bench.PARITY_BOUND
