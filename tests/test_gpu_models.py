"""Model-level parity: every layer of the benchmark graphs (at reduced sizes) against the CPU
oracle GIVEN THE DEVICE'S OWN INPUT to that layer, then fused plan == unfused plan bit for bit.

Checking each layer on the device's own input separates kernel parity (the 1e-4 bar, or
bit-exactness) from the growth of rounding differences through a deep net."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EXACT = {"batchnorm", "relu", "maxpool2d", "avgpool2d", "resize", "concat", "sum", "add_n", "pad", "reshape"}


def layer_oracle(ora, l, ins):
    k = l.kind
    if k == "conv2d":
        cd = l.attrs["cd"]
        return ora.conv2d(ins[0], l.params["K"], l.params["bias"] if cd.use_bias else None, (cd.sr, cd.sc), cd.padrt, cd.padcl,
                          cd.r, cd.c, algo="im2col")
    if k == "batchnorm":
        return ora.batchnorm_inference(ins[0], l.params["mean"], l.params["variance"], l.params.get("bn_g"), l.params.get("bn_b"),
                                       l.attrs["epsilon"])[0]
    if k == "relu":
        return ora.relu(ins[0])
    if k == "sigmoid":
        return ora.sigmoid(ins[0])
    if k == "softmax":
        return ora.softmax(ins[0], l.attrs["axis"])
    if k == "maxpool2d":
        pd = l.attrs["pd"]
        return ora.maxpool2d(ins[0], pd.ksize, pd.stride, pd.pad, fill=0.0)
    if k == "avgpool2d":
        pd = l.attrs["pd"]
        return ora.avgpool2d(ins[0], pd.ksize, pd.stride, pd.pad)
    if k == "resize":
        return ora.scale_nearest(ins[0], l.attrs["new_shape"])
    if k == "concat":
        return ora.concat(ins, l.attrs["axis"])
    if k == "sum":
        return ora.add(ins[0], ins[1])
    if k == "pad":
        return ora.pad(ins[0], l.attrs["pads"], l.attrs["constant"])
    if k == "reshape":
        return ins[0].reshape(l.out_shape)
    if k == "dense":
        return ora.dense(ins[0].reshape(-1, ins[0].shape[-1]), l.params["W"], l.params["bias"] if l.attrs["use_bias"] else None)
    raise AssertionError(k)


def table_has_upsampled_geometry(hip):
    """Whether the plan search has met a 2x2 filter on an input upsampled twice (kind 2 / 3 in the plans table): such a
    call can take a form of its own (plan tiles 8 / 9), which exists only for the fused call (UpSampling2D and Pad folded
    into the convolution), so it is searched as a geometry of its own and a fused plan that holds one agrees with the
    layer walk to the convolution's tolerance, not bit for bit."""
    import os
    import tempfile
    if hip.conv_tuned_plans() == 0:
        return False
    fd, path = tempfile.mkstemp(suffix=".txt")
    os.close(fd)
    try:
        hip.conv_tuned_save(path)
        return any(int(l.split("|")[0].split()[9]) >= 2 for l in open(path).read().splitlines() if l and not l.startswith("#"))
    finally:
        os.unlink(path)


def assert_fused_equals_walk(hip, walked, fused):
    exact = not table_has_upsampled_geometry(hip)
    for a, b in zip(walked, fused):
        if exact:
            assert np.array_equal(a, b), "fused plan differs from the layer-by-layer plan"
        else:
            assert np.abs(a - b).max() <= 1e-4 * np.abs(a).max(), "fused plan (with an upsampled 2x2 geometry) differs from the layer-by-layer plan by %g" % np.abs(a - b).max()


def check_model(hip, ora, model, x, seed):
    from eddl_amd import models
    models.init_he_normal(model, seed)
    model.build(hip, fuse=False)
    outs_unfused = [o.copy() for o in model.predict([x])]
    dev = {id(l): model.output_of(l).numpy() for l in model.layers}
    for l in model.layers:
        if l.kind == "input":
            continue
        ins = [dev[id(p)] for p in l.parents]
        ref = layer_oracle(ora, l, ins)
        got = dev[id(l)]
        if l.kind == "maxpool2d":
            ref, ix, iy = ref
            aux = model.aux[id(l)]
            assert np.array_equal(aux["indX"].numpy(), ix) and np.array_equal(aux["indY"].numpy(), iy), l.name
        ref = ref.reshape(got.shape)
        if l.kind in EXACT:
            assert np.array_equal(ref, got), l.name
        else:
            atol = 1e-5 * float(np.abs(ref).max())
            assert np.all(np.abs(ref - got) <= atol + 1e-4 * np.abs(ref)), "%s: max err %g" % (l.name, np.abs(ref - got).max())
    n_unfused = len(model.ops)
    model.build(hip, fuse=True)
    outs_fused = model.predict([x])
    assert len(model.ops) < n_unfused
    assert_fused_equals_walk(hip, outs_unfused, outs_fused)
    return outs_fused


def test_block(hip, oracle):
    from eddl_amd import models
    m = models.conv_bn_relu_pool_block(batch=4, channels=64, size=56, filters=64)
    x = np.random.default_rng(2).standard_normal((4, 64, 56, 56), dtype=np.float32)
    check_model(hip, oracle, m, x, 2)
    assert [op.kind for op in m.ops] == ["conv2d"] and "+maxpool2d" in m.ops[0].name   # the pool joins the convolution's call


def test_vgg16_small(hip, oracle):
    from eddl_amd import models
    m = models.vgg16(batch=2, size=32, num_classes=10, dense=128)
    x = np.random.default_rng(3).uniform(0, 1, (2, 3, 32, 32)).astype(np.float32)
    out = check_model(hip, oracle, m, x, 3)[0]
    np.testing.assert_allclose(out.sum(1), 1.0, rtol=1e-5)
    assert sum(op.kind == "conv2d" for op in m.ops) == 13 and not any(op.kind == "relu" and "conv" in op.name for op in m.ops)


def test_resnet50_small(hip, oracle):
    from eddl_amd import models
    m = models.resnet50(batch=2, size=64, num_classes=10, base=16)
    x = np.random.default_rng(4).standard_normal((2, 3, 64, 64), dtype=np.float32)
    check_model(hip, oracle, m, x, 4)
    kinds = [op.kind for op in m.ops]
    assert kinds.count("conv2d") == 53 and "sum" not in kinds and "batchnorm" not in kinds and "relu" not in kinds


def test_unet_small(hip, oracle):
    from eddl_amd import models
    m = models.unet(batch=1, size=64, widths=(8, 16, 32, 64), bottleneck=128)
    x = np.random.default_rng(5).uniform(0, 1, (1, 1, 64, 64)).astype(np.float32)
    check_model(hip, oracle, m, x, 5)
    kinds = [op.kind for op in m.ops]
    assert "pad" not in kinds and "batchnorm" not in kinds and "concat" not in kinds and kinds.count("conv2d") == 23


def test_fused_plan_equals_layer_walk_with_the_plan_search_on(hip, oracle):
    """The plan search keys on what a plan fixes (channels, filter, output pixels), not on paddings or the form of the input,
    so a folded Pad / Concat / UpSampling and a fused epilogue still give the layer-by-layer result bit for bit - with one
    exception: a 2x2 filter behind an UpSampling2D has a form that only the folded call can take, is searched as a geometry
    of its own, and the two then agree to the tolerance (assert_fused_equals_walk; ResNet-50 here has none and stays exact)."""
    from eddl_amd import models
    hip.conv_autotune(-1)
    try:
        hip.conv_autotune(True)
        m = models.resnet50(batch=2, size=64, num_classes=10, base=16)
        x = np.random.default_rng(4).standard_normal((2, 3, 64, 64), dtype=np.float32)
        check_model(hip, oracle, m, x, 4)
        assert not table_has_upsampled_geometry(hip)      # (so the comparison above was bit for bit)
        m = models.unet(batch=1, size=64, widths=(8, 16, 32, 64), bottleneck=128)
        x = np.random.default_rng(5).uniform(0, 1, (1, 1, 64, 64)).astype(np.float32)
        check_model(hip, oracle, m, x, 5)
        assert hip.conv_tuned_plans() > 10 and table_has_upsampled_geometry(hip)
    finally:
        hip.conv_autotune(-1)


def test_batch_resize_and_asymmetric_padding_exception(hip, oracle):
    from eddl_amd import models, net as L
    m = models.conv_bn_relu_pool_block(batch=2, channels=8, size=12, filters=8)
    models.init_he_normal(m, 9)
    m.build(hip)
    x = np.random.default_rng(9).standard_normal((5, 8, 12, 12), dtype=np.float32)
    y5 = m.predict([x])[0]          # batch 2 -> 5: every tensor re-created
    y3 = m.predict([x[:3]])[0]
    assert y5.shape == (5, 8, 6, 6) and np.array_equal(y5[:3], y3)
    with pytest.raises(L.AsymmetricPaddingException):
        L.Conv2D(L.Input([3, 224, 224], 1), 64, [7, 7], [2, 2], "same")
    with pytest.raises(L.AsymmetricPaddingException):
        L.Conv2D(L.Input([3, 8, 8], 1), 4, [2, 2], [1, 1], "same")


def test_set_parameters_after_build_reaches_the_cached_filters(hip, oracle):
    from eddl_amd import models
    m = models.conv_bn_relu_pool_block(batch=2, channels=8, size=12, filters=8)
    models.init_he_normal(m, 11)
    m.build(hip)                     # registers the convolution's filters with the library
    x = np.random.default_rng(11).standard_normal((2, 8, 12, 12), dtype=np.float32)
    y1 = m.predict([x])[0]
    params = m.get_parameters()
    models.init_he_normal(m, 12)
    m.set_parameters(m.get_parameters())
    y2 = m.predict([x])[0]
    fresh = models.conv_bn_relu_pool_block(batch=2, channels=8, size=12, filters=8)
    models.init_he_normal(fresh, 12)
    fresh.build(hip, cache_filters=False)
    assert np.array_equal(y2, fresh.predict([x])[0]) and not np.array_equal(y1, y2)
    m.set_parameters(params)
    assert np.array_equal(m.predict([x])[0], y1)


def test_predict_batches_overlapped_staging_matches_predict(hip, oracle):
    """Seven different batches through the pipelined path (pinned staging, upload and download streams, two device
    buffers) give, in order, exactly what one blocking predict per batch gives."""
    from eddl_amd import models
    m = models.unet(batch=2, size=32, widths=(4, 8), bottleneck=16)
    models.init_he_normal(m, 31)
    m.build(hip)
    rng = np.random.default_rng(31)
    batches = [rng.uniform(0, 1, (2, 1, 32, 32)).astype(np.float32) for _ in range(7)]
    want = [m.predict([x])[0] for x in batches]
    got = [outs[0] for outs in m.predict_batches(batches)]
    assert len(got) == len(want)
    for a, b in zip(want, got):
        assert np.array_equal(a, b)
    assert [o[0].shape for o in m.predict_batches([batches[0]])] == [want[0].shape]
    assert list(m.predict_batches([])) == []


def test_captured_plan_replays_bit_for_bit(hip, oracle):
    """The plan recorded once as a graph gives, on every replay, what queueing the launches one by one gives:
    several replays, each on a new input, with eager work of the same net and waits between them."""
    from eddl_amd import EddlHipError, models
    nets = [
        (models.conv_bn_relu_pool_block(batch=3, channels=16, size=20, filters=24), (3, 16, 20, 20)),
        (models.resnet50(batch=2, size=64, num_classes=10, base=16), (2, 3, 64, 64)),   # K-split launches, residual epilogues, dense
        (models.unet(batch=1, size=64, widths=(8, 16, 32, 64), bottleneck=128), (1, 1, 64, 64)),  # concat, upsampling, folded pads
        (models.vgg16(batch=2, size=32, num_classes=10, dense=128), (2, 3, 32, 32)),
    ]
    rng = np.random.default_rng(77)
    for i, (m, shape) in enumerate(nets):
        models.init_he_normal(m, 70 + i)
        for fuse in (True, False):
            m.build(hip, fuse=fuse)
            with pytest.raises(RuntimeError):
                m.run_graph()                # nothing captured yet
            m.capture()
            for _ in range(4):
                x = rng.standard_normal(shape, dtype=np.float32)
                want = m.predict([x])[0].copy()          # eager, with its waits and copies
                m.input_tensor().copy_from(rng.standard_normal(shape, dtype=np.float32))
                m.run()                                   # eager work on another input in between
                hip.synchronize()
                m.input_tensor().copy_from(x)
                m.run_graph()
                got = m.out[id(m.lout[0])].numpy()
                assert np.array_equal(got, want), (i, fuse)
    # a call that waits is refused while recording, and the recording can still be closed
    m = nets[0][0]

    def bad():
        m.run()
        hip.synchronize()
    with pytest.raises(EddlHipError, match="graph_begin and eddlhip_graph_end"):
        hip.record(bad)
    m.run()            # the device and the library are usable afterwards
    hip.synchronize()
    g = hip.record(m.run)
    g.launch()
    hip.synchronize()


def need_more_workspace(hip):
    """Run one convolution that needs more workspace than the library holds (so that it replaces it); returns the size before.
    Small workspaces: unregistered filters whose repacked copy is larger.  Beyond what a filter matrix may take (2 GiB, and
    the workspace only grows within a process): a forced Winograd form whose transformed tensors are larger."""
    ws = hip.workspace_bytes()
    if ws < (1 << 30):
        C = 64
        Kf = ((ws + (1 << 20)) // (9 * C * 4) // 128 + 1) * 128
        w, x, O = hip.full((Kf, C, 3, 3), 0.0), hip.full((1, C, 4, 4), 1.0), hip.empty((1, Kf, 4, 4))
        hip.conv2D(x, w, None, O, 1, 1, 1, 1)
    else:
        C = 16
        blocks = (ws + (64 << 20)) // (2 * 16 * C * 4) + 1   # V and M: 16 planes of C floats per 2x2 block each
        N = blocks // (128 * 128) + 1
        w, x, O = hip.full((C, C, 3, 3), 0.0), hip.full((N, C, 256, 256), 1.0), hip.empty((N, C, 256, 256))
        hip.force_conv_plan(4, 1)
        try:
            hip.conv2D(x, w, None, O, 1, 1, 1, 1)
            assert hip.last_conv_kernel().startswith("winograd")
        finally:
            hip.force_conv_plan(-1, 1)
    hip.synchronize()
    return ws


def test_recorded_graph_is_refused_after_the_workspace_was_replaced(hip):
    """A recorded convolution with unregistered filters names the library's workspace by address.  When a later,
    larger call has made the library replace that workspace, the replay is refused (not run over freed memory);
    a new recording works.  A tensor collected while recording is freed once the recording has ended."""
    from eddl_amd import EddlHipError
    rng = np.random.default_rng(5)
    x, w = hip.array(rng.standard_normal((2, 8, 12, 12), dtype=np.float32)), hip.array(rng.standard_normal((16, 8, 3, 3), dtype=np.float32))
    O = hip.empty((2, 16, 12, 12))
    box = [hip.empty((1024,))]

    def step():
        hip.conv2D(x, w, None, O, 1, 1, 1, 1)
        box.pop() if box else None  # a DeviceTensor collected while recording: its free is refused, then made up for

    hip.conv2D(x, w, None, O, 1, 1, 1, 1)
    want = O.numpy()
    g = hip.record(step)
    assert hip._deferred_free == []
    hip.fill_(O, 0.0)
    g.launch()
    assert np.array_equal(O.numpy(), want)
    # an eager convolution that needs more than the whole workspace of the moment
    ws = need_more_workspace(hip)
    assert hip.workspace_bytes() > ws
    with pytest.raises(EddlHipError, match="record again"):
        g.launch()
    g2 = hip.record(lambda: hip.conv2D(x, w, None, O, 1, 1, 1, 1))
    hip.fill_(O, 0.0)
    g2.launch()
    assert np.array_equal(O.numpy(), want)
    # a graph whose calls do not take the workspace (registered filters, no K split) stays valid
    hip.cache_conv_filters(w)
    hip.conv2D(x, w, None, O, 1, 1, 1, 1)
    g3 = hip.record(lambda: hip.conv2D(x, w, None, O, 1, 1, 1, 1))
    ws = need_more_workspace(hip)
    assert hip.workspace_bytes() > ws
    hip.fill_(O, 0.0)
    g3.launch()
    assert np.array_equal(O.numpy(), want)
    hip.uncache_conv_filters(w)


def test_bench_line_carries_the_contract_fields(hip):
    """bench.py on the smallest workload: ONE JSON line with the agreed fields, roofline and CPU baseline with its
    end-to-end parity gate; the layer-by-layer and recorded-plan modes run too."""
    import json
    import os
    import subprocess
    import sys
    from conftest import ROOT
    base = [sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "conv", "--steps", "5", "--warmup", "2", "--no-device-probe"]
    res = subprocess.run(base, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    r = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == 5 and r["warmup"] == 2 and r["dtype"] == "f32" and r["vs_baseline"] is None
    assert r["value"] > 0 and "workload" in r["config"]
    rf = r["roofline"]
    assert rf["bound"] in ("hbm", "mfma") and rf["peak"] == 157.3 and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    cb = r["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["parity"]["ok"]
    for extra in (["--unfused"], ["--graph"]):
        res = subprocess.run(base + ["--no-cpu-baseline"] + extra, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
        assert res.returncode == 0, res.stderr[-2000:]
        assert json.loads(res.stdout.strip().splitlines()[-1])["value"] > 0
