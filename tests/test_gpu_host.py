"""The C++ host layer (eddl_amd/host: Tensor, ConvolDescriptor, PoolDescriptor, gpu_*, tensorNN::*)
driven at descriptor level the way the reference's unit tests drive its seam, through a small
C++ program (tests/host/host_driver.cpp); results are compared with the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, tensor_of

pytestmark = pytest.mark.gpu

DRIVER = os.path.join(ROOT, "eddl_amd", "host", "host_driver")


def run_driver(case, tmp, params, files):
    assert os.path.exists(DRIVER), "build the host layer first: make -C eddl_amd/host"
    with open(tmp / "params.txt", "w") as fh:
        fh.write(" ".join(str(p) for p in params))
    for name, arr in files.items():
        np.ascontiguousarray(arr, np.float32).tofile(tmp / name)
    # (EDDLHIP_NO_TUNE: the binding's gpu_init would switch the plan search on; these tests compare with untuned launches bit for bit)
    res = subprocess.run([DRIVER, case, str(tmp)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120, env=dict(os.environ, EDDLHIP_NO_TUNE="1"))
    assert res.returncode == 0, res.stderr[-2000:]
    return res


def read(tmp, name):
    shape = [int(v) for v in open(tmp / (name + ".shape")).read().split()]
    return np.fromfile(tmp / (name + ".bin"), np.float32).reshape(shape)


def test_conv2d_through_descriptors(oracle, golden, tmp_path):
    for case in golden["conv2d"]:
        x = tensor_of(case["image"])
        kshape = (case["filters"], x.shape[1], *case["kernel"])
        w = np.ones(kshape, np.float32) if case["filters_data"] == "ones" else tensor_of(case["filters_data"])
        b = np.zeros(case["filters"], np.float32) if case["bias_data"] == "zeros" else tensor_of(case["bias_data"])
        run_driver("conv2d", tmp_path, [*x.shape, case["filters"], *case["kernel"], *case["strides"], int(case["use_bias"]), case["padding"]],
                   {"I.bin": x, "K.bin": w, "bias.bin": b})
        assert np.array_equal(read(tmp_path, "O"), tensor_of(case["forward"])), case["name"]
    rng = np.random.default_rng(50)
    for (N, C, H, W, Kf, R, S, sr, sc, padding, pads) in [(4, 32, 28, 28, 64, 3, 3, 1, 1, "same", None),
                                                           (2, 3, 37, 41, 16, 7, 7, 2, 2, "custom", [3, 3, 3, 3]),
                                                           (3, 5, 17, 13, 7, 3, 3, 2, 2, "same", None)]:
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
        b = rng.standard_normal(Kf, dtype=np.float32)
        run_driver("conv2d", tmp_path, [N, C, H, W, Kf, R, S, sr, sc, 1, padding] + (pads or []), {"I.bin": x, "K.bin": w, "bias.bin": b})
        P, Q, p4 = oracle.conv_geometry(H, W, R, S, sr, sc, padding, pads)
        ref = oracle.conv2d(x, w, b, (sr, sc), p4[0], p4[2], P, Q)
        out = read(tmp_path, "O")
        assert out.shape == ref.shape
        atol = 1e-5 * float(np.abs(ref).max())
        assert np.all(np.abs(ref - out) <= atol + 1e-4 * np.abs(ref))


def test_pools_through_descriptors(oracle, golden, tmp_path):
    for case in golden["maxpool2d"]:
        x = tensor_of(case["image"])
        run_driver("mpool", tmp_path, [*x.shape, *case["kernel"], *case["strides"], case["padding"]], {"I.bin": x})
        assert np.array_equal(read(tmp_path, "O"), tensor_of(case["forward"])), case["name"]
    for case in golden["avgpool2d"]:
        x = tensor_of(case["image"])
        run_driver("avgpool", tmp_path, [*x.shape, *case["kernel"], *case["strides"], case["padding"]], {"I.bin": x})
        np.testing.assert_allclose(read(tmp_path, "O"), tensor_of(case["forward"]), atol=case["atol"])
    rng = np.random.default_rng(51)
    x = rng.integers(-3, 4, size=(2, 8, 28, 28)).astype(np.float32)
    run_driver("mpool", tmp_path, [2, 8, 28, 28, 3, 3, 2, 2, "custom", 1, 1, 1, 1], {"I.bin": x})
    O, ix, iy = oracle.maxpool2d(x, (3, 3), (2, 2), (1, 1, 1, 1), fill=-1.0)
    assert np.array_equal(read(tmp_path, "O"), O) and np.array_equal(read(tmp_path, "indX"), ix) and np.array_equal(read(tmp_path, "indY"), iy)
    x = rng.standard_normal((2, 16, 7, 7), dtype=np.float32)
    run_driver("avgpool", tmp_path, [2, 16, 7, 7, 7, 7, 1, 1, "none"], {"I.bin": x})
    assert np.array_equal(read(tmp_path, "O"), oracle.avgpool2d(x, (7, 7), (1, 1), (0, 0, 0, 0)))


def test_batchnorm_and_layer_chain(oracle, tmp_path):
    rng = np.random.default_rng(52)
    N, C, H, W = 3, 6, 5, 7
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    mean = (rng.standard_normal(C) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, C).astype(np.float32)
    g = rng.uniform(0.8, 1.2, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    run_driver("bn", tmp_path, [N, C, H, W, 1e-5, 1], {"I.bin": x, "mean.bin": mean, "var.bin": var, "g.bin": g, "b.bin": b})
    y, opa, sd = oracle.batchnorm_inference(x, mean, var, g, b, 1e-5)
    assert np.array_equal(read(tmp_path, "O"), y) and np.array_equal(read(tmp_path, "opa"), opa) and np.array_equal(read(tmp_path, "bn_var"), sd)

    ndim = 10
    skip = rng.standard_normal((N, C, 2 * H + 1, 2 * W + 1), dtype=np.float32)
    feat = 2 * C * (2 * H + 1) * (2 * W + 1)
    Wd = (rng.standard_normal((feat, ndim)) * np.sqrt(2.0 / feat)).astype(np.float32)
    bd = rng.standard_normal(ndim, dtype=np.float32)
    run_driver("chain", tmp_path, [N, C, H, W, ndim], {"I.bin": x, "skip.bin": skip, "W.bin": Wd, "b.bin": bd})
    up = oracle.scale_nearest(x, (2 * H, 2 * W))
    cat = oracle.concat([skip, oracle.pad(up, (0, 1, 1, 0))], 1)
    assert np.array_equal(read(tmp_path, "cat"), cat)
    s = oracle.add(cat, cat)
    act = oracle.relu((np.zeros_like(cat) + cat) + s)
    assert np.array_equal(read(tmp_path, "act").reshape(act.shape), act)
    dense = oracle.dense(act.reshape(N, feat), Wd, bd)
    got = read(tmp_path, "dense")
    assert np.all(np.abs(dense - got) <= 1e-5 * np.abs(dense).max() + 1e-4 * np.abs(dense))
    np.testing.assert_allclose(read(tmp_path, "prob"), oracle.softmax(got, 1), rtol=2e-6, atol=1e-8)
    np.testing.assert_allclose(read(tmp_path, "sig"), oracle.sigmoid(got), rtol=1e-6, atol=1e-7)


def test_error_behaviour_follows_the_reference(tmp_path):
    res = run_driver("errors", tmp_path, [], {})
    assert "errors OK" in res.stdout
    assert "⚠️" in res.stderr  # the reference's msg() banner


# ---------------------------------------------------------------------------- model level (eddl:: API in C++)
NET_DRIVER = os.path.join(ROOT, "eddl_amd", "host", "net_driver")


def run_net_driver(args, timeout=300, env=None):
    """Runs the C++ model driver.  The binding's gpu_init switches the library's plan search on, as the reference's CUDA
    backend searches its algorithms; tests that compare with the Python host's untuned launches bit for bit switch it off
    (EDDLHIP_NO_TUNE), tests of the search pass their own environment."""
    assert os.path.exists(NET_DRIVER), "build the host layer first: make -C eddl_amd/host"
    res = subprocess.run([NET_DRIVER] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout,
                         env=dict(os.environ, **(env if env is not None else {"EDDLHIP_NO_TUNE": "1"})))
    assert res.returncode == 0, (res.stdout[-2000:], res.stderr[-2000:])
    return res.stdout


@pytest.mark.parametrize("fused", [False, True], ids=["layerwise", "fused"])
@pytest.mark.parametrize("which", ["block", "vgg16", "resnet50", "unet"])
def test_cpp_graphs_match_the_python_runner_bit_for_bit(hip, which, fused, tmp_path):
    """The same graph built through the C++ eddl:: API and through eddl_amd.net, the same parameters
    (written by Net.save in the reference's bin format, read by the C++ Net::load), the same input:
    identical layer order and identical outputs, after the C++ net has also been through a batch
    resize.  With Net::fuse() the C++ net runs its fused plan (parameters loaded after the plan was
    made, so the kept filter copies have to follow them) and must still give the layer-by-layer
    result of the Python runner bit for bit."""
    from eddl_amd import models
    batch = 3
    if which == "block":
        m, size, extra = models.conv_bn_relu_pool_block(batch=batch, channels=6, size=16, filters=8), 16, [6, 8]
    elif which == "vgg16":
        m, size, extra = models.vgg16(batch=batch, size=32, num_classes=10, widths=(8, 16, 16, 32, 32), dense=64), 32, [10, 8, 16, 16, 32, 32, 64]
    elif which == "resnet50":
        m, size, extra = models.resnet50(batch=batch, size=64, num_classes=10, base=8), 64, [10, 8]
    else:
        m, size, extra = models.unet(batch=batch, size=32, widths=(4, 8), bottleneck=16), 32, [4, 8, 16]
    models.init_he_normal(m, 41)
    m.save(str(tmp_path / "params.bin"))
    rng = np.random.default_rng(41)
    x = rng.standard_normal(m.lin[0].out_shape, dtype=np.float32)
    x.tofile(tmp_path / "x.raw")
    out = run_net_driver([("fused:" if fused else "") + which, tmp_path / "params.bin", tmp_path / "x.raw", tmp_path / "y.raw", batch, size] + extra)
    assert "FAILED" not in out and "ok  get_parameters / set_parameters round trip" in out and "ok  set_parameters with a missing layer" in out, out
    # the reference's host profile (eddl::show_profile): forward is counted in both modes, the dispatchers of the layer walk
    # only when the layers are walked
    prof = {l.split(":")[0].strip("| "): int(l.split(":")[1].split("calls")[0]) for l in out.splitlines() if l.startswith("| ") and " calls," in l}
    assert prof.get("forward", 0) >= 1, out
    assert ("Conv2D" in prof) == (not fused), prof
    if fused:
        assert "ok  getOutput of a fused-away layer" in out, out
        steps = int([l for l in out.splitlines() if l.startswith("plan:")][0].split()[1])
        m.build(hip, fuse=True)
        views = sum(1 for l in m.layers if l.kind in ("input", "reshape"))   # steps of the C++ plan that launch nothing
        assert steps == len(m.ops) + views, (steps, len(m.ops), views)
    kinds = [l for l in out.splitlines() if l.startswith("layers:")][0].split()[1:]
    rename = {"input": "input", "relu": "relu", "sigmoid": "sigmoid", "softmax": "softmax"}
    assert kinds == [rename.get(l.kind, l.kind) for l in m.layers], "layer order differs"
    m.build(hip, fuse=False)
    want = m.predict([x])[0]
    got = np.fromfile(tmp_path / "y.raw", np.float32).reshape(want.shape)
    assert np.array_equal(got, want)


def test_cpp_host_runs_the_plans_a_python_process_saved(hip, tmp_path):
    """Plans travel between processes as a file: the Python host searches a block's convolution once, and the file it saves
    is rewritten, to an undivided plan, to a four-way K-split and to the folded Winograd form (so that the plan in force is
    known; under the last the block's max-pool is computed in the convolution's epilogue).  The C++ host started with any of
    the files must give what the Python host gives with that file, bit for bit; the plans sum in different orders, so
    their results differ from each other in their last bits."""
    from eddl_amd import models
    batch, ch, size = 3, 64, 28
    m = models.conv_bn_relu_pool_block(batch=batch, channels=ch, size=size, filters=ch)
    models.init_he_normal(m, 43)
    m.save(str(tmp_path / "params.bin"))
    x = np.random.default_rng(43).standard_normal(m.lin[0].out_shape, dtype=np.float32)
    x.tofile(tmp_path / "x.raw")
    plans = str(tmp_path / "plans.txt")
    assert os.path.exists(NET_DRIVER), "build the host layer first: make -C eddl_amd/host"
    want = {}
    hip.conv_autotune(-1)
    try:
        m.build(hip, fuse=True)
        hip.conv_autotune(True)
        m.predict([x])
        assert hip.conv_tuned_plans() in (1, 2)      # the convolution, and the product launch of its Winograd form
        hip.conv_tuned_save(plans)
        lines = open(plans).read().splitlines()
        keys = [l.split("|")[0] for l in lines if l and not l.startswith("#")]
        keys = [k for k in keys if k.split()[:5] == [str(batch), str(ch), str(ch), "3", "3"]]
        assert len(keys) == 1, lines
        for plan in ("2 1", "2 4", "5 1"):          # 5: the folded Winograd form, which also pools in its own epilogue
            with open(plans + plan.replace(" ", "_"), "w") as f:
                f.write("# rewritten by the test\n" + keys[0] + "| " + plan + "\n")
            hip.conv_autotune(-1)
            hip.conv_tuned_load(plans + plan.replace(" ", "_"))
            hip.conv_autotune(True)
            want[plan] = m.predict([x])[0]
            assert hip.last_conv_kernel().startswith("winograd") == (plan == "5 1")
    finally:
        hip.conv_autotune(-1)
    assert not np.array_equal(want["2 1"], want["2 4"]) and np.allclose(want["2 1"], want["2 4"], rtol=1e-4, atol=1e-5)
    assert not np.array_equal(want["2 1"], want["5 1"]) and np.allclose(want["2 1"], want["5 1"], rtol=1e-4, atol=1e-5)
    for plan in want:
        res = subprocess.run([NET_DRIVER, "fused:block", str(tmp_path / "params.bin"), str(tmp_path / "x.raw"), str(tmp_path / "y.raw"), str(batch), str(size), str(ch), str(ch)],
                             stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300, env=dict(os.environ, EDDLHIP_PLANS=plans + plan.replace(" ", "_")))
        assert res.returncode == 0 and "plans: 1 geometries loaded" in res.stdout and "FAILED" not in res.stdout, (res.stdout[-2000:], res.stderr[-2000:])
        got = np.fromfile(tmp_path / "y.raw", np.float32).reshape(want[plan].shape)
        assert np.array_equal(got, want[plan]), plan


@pytest.mark.parametrize("fused", [False, True], ids=["layerwise", "fused"])
def test_cpp_host_searches_its_plans_like_the_reference_backend(hip, fused, tmp_path):
    """An unchanged EDDL program gets the plan search: the binding's gpu_init switches it on (the reference's gpu_conv2D
    runs cudnnFindConvolutionForwardAlgorithm on a layer's first forward).  A VGG-shaped net (channels in sixteens, so every
    Winograd form is a candidate) walked layer by layer, and as its fused plan, by the C++ host with nothing in its
    environment; the table it ends up with is saved, and the Python layer walk under that table gives the same bits."""
    from eddl_amd import models
    batch, size, extra = 4, 64, [10, 16, 32, 64, 64, 64, 64]
    m = models.vgg16(batch=batch, size=size, num_classes=10, widths=(16, 32, 64, 64, 64), dense=64)
    models.init_he_normal(m, 4)
    x = models.synthetic_input(m.lin[0].out_shape, 1004, "uniform")
    plans = str(tmp_path / "plans.txt")
    out = run_net_driver([("fused:" if fused else "") + "vgg16", "synth:4", "synth:1004:uniform", tmp_path / "y.raw", batch, size] + extra,
                         env={"EDDLHIP_PLANS_SAVE": plans, "EDDLHIP_NO_TUNE": ""})
    assert "FAILED" not in out, out
    searched = [l for l in open(plans).read().splitlines() if l and not l.startswith("#")]
    assert len(searched) >= 8, searched          # batch 1 (the driver's resize) and batch 4 geometries
    hip.conv_autotune(-1)
    try:
        hip.conv_tuned_load(plans)
        hip.conv_autotune(True)
        m.build(hip, fuse=False)
        want = m.predict([x])[0]
        assert hip.conv_tuned_plans() == len(searched)      # nothing was left to search
    finally:
        hip.conv_autotune(-1)
    got = np.fromfile(tmp_path / "y.raw", np.float32).reshape(want.shape)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("which", ["block", "resnet50", "unet"])
def test_cpp_host_builds_a_configuration_from_seeds_alone(hip, which, tmp_path):
    """No parameter file and no input file: the C++ host draws both from the generator it shares with the Python host
    (mt19937 + Box-Muller, seeds as the benchmark uses them) and must produce what the Python graph produces."""
    from eddl_amd import models
    batch = 2
    if which == "block":
        m, size, extra, dist = models.conv_bn_relu_pool_block(batch=batch, channels=6, size=16, filters=8), 16, [6, 8], "normal"
    elif which == "resnet50":
        m, size, extra, dist = models.resnet50(batch=batch, size=64, num_classes=10, base=8), 64, [10, 8], "normal"
    else:
        m, size, extra, dist = models.unet(batch=batch, size=32, widths=(4, 8), bottleneck=16), 32, [4, 8, 16], "uniform"
    models.init_he_normal(m, 4)
    x = models.synthetic_input(m.lin[0].out_shape, 1004, dist)
    out = run_net_driver(["fused:" + which, "synth:4", "synth:1004:" + dist, tmp_path / "y.raw", batch, size] + extra)
    assert "FAILED" not in out, out
    m.build(hip, fuse=False)
    want = m.predict([x])[0]
    got = np.fromfile(tmp_path / "y.raw", np.float32).reshape(want.shape)
    assert np.array_equal(got, want)


def test_cpp_graph_errors_and_parameter_round_trip(hip, tmp_path):
    out = run_net_driver(["errors"])
    assert "FAILED" not in out and out.count("ok ") >= 17, out
    # freshly initialised parameters saved by the C++ net load into the Python graph and give the same output
    from eddl_amd import models
    m = models.conv_bn_relu_pool_block(batch=2, channels=5, size=12, filters=7)
    x = np.random.default_rng(42).standard_normal((2, 5, 12, 12), dtype=np.float32)
    x.tofile(tmp_path / "x.raw")
    run_net_driver(["block", "-", tmp_path / "x.raw", tmp_path / "y.raw", 2, 12, 5, 7])
    m.load(str(tmp_path / "y.raw.params"))
    K = [l for l in m.layers if l.kind == "conv2d"][0].params["K"]
    assert K.std() > 0 and np.abs(K).max() <= np.sqrt(6.0 / (5 * 9 + 7 * 9)) + 1e-6   # Glorot-uniform range
    m.build(hip, fuse=False)
    want = m.predict([x])[0]
    assert np.array_equal(np.fromfile(tmp_path / "y.raw", np.float32).reshape(want.shape), want)


# ---------------------------------------------------------------------------- ONNX through the C++ host layer
@pytest.mark.parametrize("fused", [0, 1], ids=["layerwise", "fused"])
@pytest.mark.parametrize("name", ["vgg_like", "resnet_like", "unet_like"])
def test_cpp_onnx_import_matches_pytorch_and_the_python_importer(hip, name, fused, tmp_path):
    """The files PyTorch wrote (tests/golden/onnx), imported by the C++ import_net_from_onnx_file: same
    layers and names as the Python importer builds, PyTorch's outputs within the convolution tolerance,
    the Python runner's outputs bit for bit; the net written back by the C++ exporter loads in the
    Python importer with identical layers and parameters."""
    from eddl_amd import onnx_io
    fix = os.path.join(ROOT, "tests", "golden", "onnx")
    d = np.load(os.path.join(fix, name + ".npz"))
    d["x"].tofile(tmp_path / "x.raw")
    out = run_net_driver(["onnx", os.path.join(fix, name + ".onnx"), tmp_path / "x.raw", tmp_path / "y.raw", d["x"].shape[0], fused,
                          tmp_path / "back.onnx"])
    assert "FAILED" not in out and "ok  missing ONNX file" in out, out
    net = onnx_io.import_net_from_onnx_file(os.path.join(fix, name + ".onnx"))
    kinds = [l for l in out.splitlines() if l.startswith("layers:")][0].split()[1:]
    names = [l for l in out.splitlines() if l.startswith("names:")][0].split()[1:]
    assert kinds == [l.kind for l in net.layers] and names == [l.name for l in net.layers]
    got = np.fromfile(tmp_path / "y.raw", np.float32).reshape(d["y"].shape)
    assert np.all(np.abs(got - d["y"]) <= 1e-5 * np.abs(d["y"]).max() + 1e-4 * np.abs(d["y"]))
    net.build(hip, fuse=False)
    assert np.array_equal(got, net.predict([d["x"]])[0])
    back = onnx_io.import_net_from_onnx_file(str(tmp_path / "back.onnx"))
    assert [(l.kind, l.name, l.out_shape[1:]) for l in back.layers] == [(l.kind, l.name, l.out_shape[1:]) for l in net.layers]
    for a, b in zip(net.layers, back.layers):
        for key in a.params:
            if key == "bias" and not (a.attrs["cd"].use_bias if a.kind == "conv2d" else a.attrs.get("use_bias", True)):
                continue
            assert np.array_equal(a.params[key], b.params[key]), (a.name, key)


@pytest.mark.parametrize("seed", range(12))
def test_cpp_fused_plan_on_random_graphs(hip, seed, tmp_path):
    """Random graphs (tests/test_onnx_cpu.py:random_net) written to ONNX, imported by the C++ host layer and
    run through Net::fuse: bit for bit what the Python layer walk computes, so the C++ chain rules
    (pad folding, batch norm, LSum / LAdd + ReLU, dense + ReLU) hold on graphs nobody wrote by hand."""
    from eddl_amd import onnx_io
    from test_onnx_cpu import random_net
    rng = np.random.default_rng(900 + seed)
    data = onnx_io.export_net_to_onnx_bytes(random_net(rng))
    (tmp_path / "g.onnx").write_bytes(data)
    net = onnx_io.import_net_from_onnx_bytes(data)
    x = rng.standard_normal([3] + net.lin[0].out_shape[1:]).astype(np.float32)
    x.tofile(tmp_path / "x.raw")
    for fused in (0, 1):
        out = run_net_driver(["onnx", tmp_path / "g.onnx", tmp_path / "x.raw", tmp_path / ("y%d.raw" % fused), 3, fused])
        assert "FAILED" not in out, out
    net.build(hip, fuse=False)
    want = net.predict([x])[0]
    for fused in (0, 1):
        got = np.fromfile(tmp_path / ("y%d.raw" % fused), np.float32).reshape(want.shape)
        assert np.array_equal(got, want), (fused, np.abs(got - want).max())
