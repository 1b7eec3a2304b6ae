"""Parity of the HIP kernels, called through the C ABI, with the CPU oracle on the same
seeded inputs, and with the vectors the reference's own tests hold.

Bars: bit-exact for ReLU, Add, Concat, UpSampling, Pad, MaxPool (values and argmax indices),
AvgPool, BatchNorm-inference and the scalar direct convolution; floating-point tolerance for
the MFMA convolution (|a-b| <= atol + rtol*|b|, rtol 1e-4, atol 1e-5*max|ref|), dense,
sigmoid and softmax (different summation order / exp implementation).
"""
import numpy as np
import pytest

from conftest import eddl_allclose, tensor_of

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def assert_conv_close(ref, out, what=""):
    atol = 1e-5 * float(np.max(np.abs(ref)))
    err = np.abs(ref - out) - (atol + RTOL * np.abs(ref))
    assert np.all(err <= 0), "%s: worst excess %g at %s (ref %g out %g)" % (
        what, err.max(), np.unravel_index(err.argmax(), err.shape), ref.flat[err.argmax()], out.flat[err.argmax()])


def run_conv(hip, oracle, x, w, b, stride, padding, pads=None, algo="auto", bn=None, residual=None, relu=False):
    from eddl_amd.descriptors import ConvolDescriptor
    cd = ConvolDescriptor(w.shape[0], list(w.shape[2:]), list(stride), padding, pads or [], use_bias=b is not None).build(list(x.shape))
    O = hip.empty(cd.out_shape)
    dbn = None
    if bn is not None:
        g, bb, mean, var, eps = bn
        dbn = (hip.array(g) if g is not None else None, hip.array(bb) if bb is not None else None, hip.array(mean), hip.array(var), eps)
    hip.set_conv_algo(algo)
    try:
        hip.conv2D(hip.array(x), hip.array(w), hip.array(b) if b is not None else None, O, cd.sr, cd.sc, cd.padrt, cd.padcl,
                   bn=dbn, residual=hip.array(residual) if residual is not None else None, relu=relu)
    finally:
        hip.set_conv_algo("auto")
    ref = oracle.conv2d(x, w, b, stride, cd.padrt, cd.padcl, cd.r, cd.c)
    if bn is not None:
        g, bb, mean, var, eps = bn
        ref, _, _ = oracle.batchnorm_inference(ref, mean, var, g, bb, eps)
    if residual is not None:
        ref = oracle.add(ref, residual)
    if relu:
        ref = oracle.relu(ref)
    return ref, O.numpy()


# ------------------------------------------------------------------ reference-held vectors
def _conv_inputs(case):
    x = tensor_of(case["image"])
    kshape = (case["filters"], x.shape[1], case["kernel"][0], case["kernel"][1])
    w = np.ones(kshape, np.float32) if case["filters_data"] == "ones" else tensor_of(case["filters_data"])
    b = np.zeros(case["filters"], np.float32) if case["bias_data"] == "zeros" else tensor_of(case["bias_data"])
    return x, w, (b if case["use_bias"] else None)


@pytest.mark.parametrize("algo", ["mfma_staged", "mfma_lds", "direct"])
def test_conv2d_reference_vectors(hip, oracle, golden, algo):
    for case in golden["conv2d"]:
        x, w, b = _conv_inputs(case)
        ref, out = run_conv(hip, oracle, x, w, b, case["strides"], case["padding"], algo=algo)
        exp = tensor_of(case["forward"])
        assert out.shape == exp.shape, case["name"]
        assert eddl_allclose(exp, out, case["atol"], case["rtol"]), case["name"]
        assert np.array_equal(exp, out), case["name"]  # small integers: exact in any order


def test_pool_reference_vectors(hip, golden):
    from eddl_amd.descriptors import PoolDescriptor
    for case in golden["maxpool2d"]:
        x = tensor_of(case["image"])
        pd = PoolDescriptor(case["kernel"], case["strides"], case["padding"]).build(list(x.shape))
        O, ix, iy = hip.empty(pd.out_shape), hip.full(pd.out_shape, -1.0), hip.full(pd.out_shape, -1.0)
        hip.mpool2D(hip.array(x), O, ix, iy, pd.ksize, pd.stride, pd.pad)
        assert np.array_equal(O.numpy(), tensor_of(case["forward"])), case["name"]
        hist = np.zeros_like(x)
        for yy, xx in zip(iy.numpy().ravel(), ix.numpy().ravel()):
            hist[0, 0, int(yy), int(xx)] += 1
        assert np.array_equal(hist, tensor_of(case["backward_of_ones"])), case["name"]
    for case in golden["avgpool2d"]:
        x = tensor_of(case["image"])
        pd = PoolDescriptor(case["kernel"], case["strides"], case["padding"]).build(list(x.shape))
        O = hip.empty(pd.out_shape)
        hip.avgpool2D(hip.array(x), O, pd.ksize, pd.stride, pd.pad)
        assert eddl_allclose(tensor_of(case["forward"]), O.numpy(), case["atol"], case["rtol"]), case["name"]


def test_pad_and_softmax_reference_vectors(hip, golden):
    case = golden["pad"]
    x = tensor_of(case["input"])
    exp = tensor_of(case["expected"])
    B = hip.full(exp.shape, 0.0)
    hip.pad(hip.array(x), B, case["pads"])
    assert eddl_allclose(exp, B.numpy(), case["atol"])
    case = golden["softmax"]
    x = tensor_of(case["input"])
    B = hip.empty(x.shape)
    hip.full_softmax(hip.array(x), B, case["axis"])
    assert eddl_allclose(tensor_of(case["expected"]), B.numpy(), case["atol"])


# ------------------------------------------------------------------ convolution
CONV_SHAPES = [
    # N, C, H, W, Kf, R, S, sr, sc, padding, pads, bias
    (8, 3, 32, 32, 32, 3, 3, 1, 1, "same", None, True),        # the single-convolution configuration
    (2, 64, 28, 28, 64, 3, 3, 1, 1, "same", None, False),
    (2, 16, 19, 23, 130, 3, 3, 1, 1, "same", None, True),      # ragged: channels and pixels not tile multiples
    (3, 5, 17, 13, 7, 3, 3, 2, 2, "same", None, True),         # asymmetric same pads
    (2, 3, 37, 41, 16, 7, 7, 2, 2, "custom", [3, 3, 3, 3], False),  # ResNet stem geometry
    (2, 32, 14, 14, 96, 1, 1, 1, 1, "valid", None, False),     # 1x1
    (2, 32, 15, 15, 48, 1, 1, 2, 2, "valid", None, True),      # 1x1 stride 2 (projection shortcut)
    (2, 8, 12, 12, 4, 2, 2, 1, 1, "valid", None, True),        # 2x2 valid (U-Net up-conv after Pad)
    (1, 64, 9, 9, 1, 1, 1, 1, 1, "valid", None, True),         # single output channel
    (2, 6, 10, 12, 5, 3, 2, 1, 2, "same", None, True),         # rectangular filter, mixed strides
    (1, 300, 8, 8, 33, 3, 3, 1, 1, "same", None, False),       # many taps (C*R*S = 2700)
    (1, 1, 64, 64, 64, 3, 3, 1, 1, "same", None, True),        # single input channel (U-Net first layer)
    (8, 32, 56, 56, 128, 3, 3, 1, 1, "same", None, True),      # enough tiles for the 128x128 kernel
    (8, 31, 56, 56, 130, 3, 3, 1, 1, "same", None, False),     # 128x128 kernel, odd channels, ragged filters
    (8, 24, 56, 56, 64, 3, 3, 1, 1, "same", None, True),       # 64x128 kernel
    (8, 40, 56, 56, 256, 1, 1, 1, 1, "valid", None, True),     # 1x1 on the 128x128 kernel, channels not a multiple of 16
    (8, 16, 57, 57, 128, 2, 2, 1, 1, "valid", None, True),     # 2x2 on the 128x128 kernel
    (6, 10, 64, 64, 16, 3, 3, 2, 2, "custom", [1, 1, 1, 1], True),  # 32x128 kernel, stride 2
]


@pytest.mark.parametrize("algo", ["mfma_staged", "mfma_lds"])
@pytest.mark.parametrize("shape", CONV_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:9]) + "-" + s[9])
def test_conv2d_mfma_against_oracle(hip, oracle, shape, algo):
    N, C, H, W, Kf, R, S, sr, sc, padding, pads, use_bias = shape
    rng = np.random.default_rng(100 + C * 7 + Kf)
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
    b = rng.standard_normal(Kf, dtype=np.float32) if use_bias else None
    ref, out = run_conv(hip, oracle, x, w, b, (sr, sc), padding, pads, algo=algo)
    assert out.shape == ref.shape
    assert_conv_close(ref, out, str(shape) + " " + hip.last_conv_kernel())


@pytest.mark.parametrize("kf", [1, 2, 3, 4])
def test_conv2d_onto_few_filters_is_the_direct_form_bit_for_bit(hip, oracle, kf):
    """A 1x1 stride-1 convolution onto at most four filters takes the streaming kernel, which adds the products in
    increasing channel order with a separate multiply and add: the reference's direct form for a one-tap filter
    (src/hardware/cpu/nn/cpu_conv.cpp:296-311).  Whole fused tail, odd channel counts, planes of a multiple of four
    pixels (16-byte accesses) and not."""
    rng = np.random.default_rng(600 + kf)
    for N, C, H, W in ((3, 64, 16, 12), (2, 5, 7, 9), (1, 13, 1, 1), (4, 8, 32, 32)):
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = rng.standard_normal((kf, C, 1, 1), dtype=np.float32)
        b = rng.standard_normal(kf).astype(np.float32)
        bn = (rng.uniform(0.8, 1.2, kf).astype(np.float32), rng.standard_normal(kf).astype(np.float32),
              rng.standard_normal(kf).astype(np.float32), rng.uniform(0.5, 1.5, kf).astype(np.float32), 1e-5)
        res = rng.standard_normal((N, kf, H, W), dtype=np.float32)
        for kw in ({}, dict(bn=bn, residual=res, relu=True)):
            ref, out = run_conv(hip, oracle, x, w, b, (1, 1), "valid", **kw)
            assert hip.last_conv_kernel().startswith("conv_pointwise_few_kernel<%d," % kf), hip.last_conv_kernel()
            assert np.array_equal(ref, out), (kf, (N, C, H, W), kw.keys())
    # the same layer through the matrix-core kernels (forced plan) agrees to the convolution tolerance
    hip.force_conv_plan(3, 1)
    try:
        ref, out = run_conv(hip, oracle, x, w, b, (1, 1), "valid")
    finally:
        hip.force_conv_plan(-1, 1)
    assert hip.last_conv_kernel().startswith("conv_tap_kernel")
    assert_conv_close(ref, out, "few filters through the tile kernel")


@pytest.mark.parametrize("shape", CONV_SHAPES[:6], ids=lambda s: "x".join(str(v) for v in s[:9]))
def test_conv2d_direct_kernel_is_bit_exact(hip, oracle, shape):
    N, C, H, W, Kf, R, S, sr, sc, padding, pads, use_bias = shape
    rng = np.random.default_rng(200 + C)
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = rng.standard_normal((Kf, C, R, S), dtype=np.float32)
    b = rng.standard_normal(Kf, dtype=np.float32) if use_bias else None
    ref, out = run_conv(hip, oracle, x, w, b, (sr, sc), padding, pads, algo="direct")
    assert np.array_equal(ref, out)


def _bn_params(rng, C):
    mean = (rng.standard_normal(C) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, C).astype(np.float32)
    g = rng.uniform(0.8, 1.2, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    return g, b, mean, var, 1e-5


def test_conv2d_fused_epilogue(hip, oracle):
    rng = np.random.default_rng(300)
    N, C, H, W, Kf = 2, 24, 14, 14, 40
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    bias = rng.standard_normal(Kf, dtype=np.float32)
    res = rng.standard_normal((N, Kf, H, W), dtype=np.float32)
    bn = _bn_params(rng, Kf)
    # direct kernel + fused tail: every step has the oracle's rounding, so it is bit-exact
    for kw in (dict(bn=bn, relu=True), dict(bn=bn, residual=res, relu=True), dict(b=bias, bn=(None, None) + bn[2:]),
               dict(b=bias, residual=res), dict(relu=True)):
        b = kw.pop("b", None)
        ref, out = run_conv(hip, oracle, x, w, b, (1, 1), "same", algo="direct", **kw)
        assert np.array_equal(ref, out), kw.keys()
    for algo in ("mfma_staged", "mfma_lds"):
        for kw in (dict(bn=bn, relu=True), dict(bn=bn, residual=res, relu=True)):
            ref, out = run_conv(hip, oracle, x, w, None, (1, 1), "same", algo=algo, **kw)
            assert_conv_close(ref, out, "fused " + algo)
            assert np.all(out >= 0)


def test_conv2d_ksplit_of_the_last_round(hip, oracle):
    """Tiles of a mostly idle last round are divided along K and added in slice order: same
    tolerance, reproducible bit for bit from run to run, and the undivided plan is still there."""
    rng = np.random.default_rng(302)
    split_seen = 0
    for (N, C, H, W, Kf, R) in [(8, 64, 28, 28, 128, 3), (4, 256, 14, 14, 256, 1), (3, 96, 20, 20, 200, 3), (32, 512, 14, 14, 512, 3)]:
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, R, R)) * np.sqrt(2.0 / (C * R * R))).astype(np.float32)
        b = rng.standard_normal(Kf, dtype=np.float32)
        outs = {}
        for mode in ("ksplit_on", "ksplit_off"):
            hip.set_conv_algo(mode)
            try:
                ref, out = run_conv(hip, oracle, x, w, b, (1, 1), "same", algo="mfma", relu=True)
                name = hip.last_conv_kernel()
                _, again = run_conv(hip, oracle, x, w, b, (1, 1), "same", algo="mfma", relu=True)
            finally:
                hip.set_conv_algo("ksplit_on")
            assert mode == "ksplit_on" or "+ksplit" not in name, name
            split_seen += "+ksplit" in name
            assert_conv_close(ref, out, name)
            assert np.array_equal(out, again), "not reproducible: " + name
            outs[mode] = out
        np.testing.assert_allclose(outs["ksplit_on"], outs["ksplit_off"], rtol=1e-4, atol=1e-4)
    assert split_seen >= 1, "the planner never divided a last round along K"


@pytest.mark.parametrize("algo", ["mfma_staged", "mfma_lds"])
def test_conv2d_every_tile_shape_and_slice_count(hip, oracle, algo):
    """The planner's choices are overridden so that every kernel variant (4 tile shapes x filter
    families 3x3, 1x1, 2x2, general) runs, divided along K and undivided, on ragged shapes."""
    rng = np.random.default_rng(303)
    shapes = [(3, 21, 20, 23, 130, 3, 3, "same"), (3, 37, 20, 23, 70, 1, 1, "valid"), (2, 10, 21, 22, 40, 2, 2, "valid"),
              (2, 9, 19, 17, 33, 3, 2, "same")]
    for (N, C, H, W, Kf, R, S, padding) in shapes:
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
        b = rng.standard_normal(Kf, dtype=np.float32)
        for tile in range(4):
            for slices in (1, 3):
                hip.force_conv_plan(tile, slices)
                try:
                    ref, out = run_conv(hip, oracle, x, w, b, (1, 1), padding, algo=algo, relu=True)
                    name = hip.last_conv_kernel()
                finally:
                    hip.force_conv_plan(-1, 1)
                assert ("+ksplit" in name) == (slices > 1), name
                assert_conv_close(ref, out, "%s tile %d slices %d: %s" % ((N, C, H, W, Kf, R, S), tile, slices, name))


@pytest.mark.parametrize("algo", ["mfma_staged", "mfma_lds", "direct"])
def test_conv2d_two_tensor_input_equals_conv_of_the_concatenation(hip, oracle, algo):
    """A channel Concat folded into the convolution: channels from two tensors give, bit for bit, what the same
    kernel gives on the concatenated tensor - 3x3, 1x1 and 2x2 filters, every tile shape, divided along K and not,
    odd half-channel counts (a K-step that takes channels from both tensors), strides, padding, the fused epilogue."""
    from eddl_amd import EddlHipError
    rng = np.random.default_rng(305)
    cases = [(3, 21, 20, 23, 70, 3, 3, 1, 1), (2, 64, 18, 18, 130, 3, 3, 1, 1), (2, 9, 21, 22, 40, 2, 2, 1, 0), (3, 37, 20, 23, 70, 1, 1, 1, 0),
             (2, 5, 15, 17, 33, 3, 3, 2, 1), (1, 1, 9, 9, 4, 3, 3, 1, 1)]
    for (N, Ch, H, W, Kf, R, S, st, pad) in cases:
        a = rng.standard_normal((N, Ch, H, W), dtype=np.float32)
        b = rng.standard_normal((N, Ch, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, 2 * Ch, R, S)) * np.sqrt(1.0 / (Ch * R * S))).astype(np.float32)
        bias = rng.standard_normal(Kf, dtype=np.float32)
        P, Q = (H + 2 * pad - R) // st + 1, (W + 2 * pad - S) // st + 1
        res = rng.standard_normal((N, Kf, P, Q), dtype=np.float32)
        g, bb, mean, var, eps = _bn_params(rng, Kf)
        A, B, AB = hip.array(a), hip.array(b), hip.array(np.concatenate([a, b], axis=1))
        Wd, Bd, Rd = hip.array(w), hip.array(bias), hip.array(res)
        bn = (hip.array(g), hip.array(bb), hip.array(mean), hip.array(var), eps)
        hip.set_conv_algo(algo)
        try:
            plans = [(-1, 1)] if algo == "direct" else [(-1, 1)] + [(t, sl) for t in range(4) for sl in (1, 3)]
            for tile, slices in plans:
                hip.force_conv_plan(tile, slices)
                for kw in (dict(), dict(bn=bn, residual=Rd, relu=True)):
                    O1, O2 = hip.empty((N, Kf, P, Q)), hip.empty((N, Kf, P, Q))
                    hip.conv2D(AB, Wd, Bd, O1, st, st, pad, pad, **kw)
                    name = hip.last_conv_kernel()
                    hip.conv2D(A, Wd, Bd, O2, st, st, pad, pad, second=B, **kw)
                    assert hip.last_conv_kernel() == name
                    assert np.array_equal(O1.numpy(), O2.numpy()), ((N, Ch, H, W, Kf, R, S), name, sorted(kw))
        finally:
            hip.force_conv_plan(-1, 1)
            hip.set_conv_algo("auto")
        ref = oracle.conv2d(np.concatenate([a, b], axis=1), w, bias, (st, st), pad, pad, P, Q)
        O = hip.empty((N, Kf, P, Q))
        hip.conv2D(A, Wd, Bd, O, st, st, pad, pad, second=B)
        assert_conv_close(ref, O.numpy(), "two tensors vs oracle %s" % ((N, Ch, H, W, Kf, R, S),))
    # other filter shapes are refused: the caller concatenates first
    a = hip.array(rng.standard_normal((1, 4, 12, 12), dtype=np.float32))
    w5 = hip.array(rng.standard_normal((6, 8, 5, 5), dtype=np.float32))
    with pytest.raises(EddlHipError, match="concatenate first"):
        hip.conv2D(a, w5, None, hip.empty((1, 6, 8, 8)), 1, 1, 0, 0, second=a)


@pytest.mark.parametrize("algo", ["mfma_staged", "mfma_lds", "direct"])
def test_conv2d_upsampled_input_equals_conv_of_the_resized_tensor(hip, oracle, algo):
    """Nearest UpSampling2D by whole factors folded into the gather: bit for bit what the same kernel gives on the
    tensor the resize kernel writes - the decoder shape (x2, zero pad right/bottom, 2x2 valid), 3x3 same, 1x1,
    unequal factors, strides, every tile shape, divided along K and not."""
    from eddl_amd import EddlHipError
    rng = np.random.default_rng(306)
    # N, C, H, W, Kf, R, S, stride, (pad_top, pad_left), (extra bottom, extra right), (uh, uw)
    cases = [(2, 24, 9, 11, 20, 2, 2, 1, (0, 0), (1, 1), (2, 2)), (3, 21, 10, 12, 70, 3, 3, 1, (1, 1), (1, 1), (2, 2)),
             (2, 37, 7, 9, 40, 1, 1, 1, (0, 0), (0, 0), (3, 2)), (2, 64, 8, 8, 130, 3, 3, 2, (1, 1), (1, 1), (2, 3)),
             (1, 3, 5, 6, 4, 3, 3, 1, (1, 1), (1, 1), (1, 4))]
    for (N, C, H, W, Kf, R, S, st, (pt, pl), (pb, pr), (uh, uw)) in cases:
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
        bias = rng.standard_normal(Kf, dtype=np.float32)
        Hu, Wu = H * uh, W * uw
        P, Q = (Hu + pt + pb - R) // st + 1, (Wu + pl + pr - S) // st + 1
        X, Wd, Bd = hip.array(x), hip.array(w), hip.array(bias)
        XU = hip.empty((N, C, Hu, Wu))
        hip.scale(X, XU, (Hu, Wu))
        assert np.array_equal(XU.numpy(), oracle.scale_nearest(x, (Hu, Wu)))
        hip.set_conv_algo(algo)
        try:
            plans = [(-1, 1)] if algo == "direct" else [(-1, 1)] + [(t, sl) for t in range(4) for sl in (1, 3)]
            for tile, slices in plans:
                hip.force_conv_plan(tile, slices)
                O1, O2 = hip.empty((N, Kf, P, Q)), hip.empty((N, Kf, P, Q))
                hip.conv2D(XU, Wd, Bd, O1, st, st, pt, pl, relu=True)
                name = hip.last_conv_kernel()
                hip.conv2D(X, Wd, Bd, O2, st, st, pt, pl, relu=True, upsample=(uh, uw))
                assert hip.last_conv_kernel() == name
                assert np.array_equal(O1.numpy(), O2.numpy()), ((N, C, H, W, Kf, R, S, uh, uw), name)
        finally:
            hip.force_conv_plan(-1, 1)
            hip.set_conv_algo("auto")
    x = hip.array(rng.standard_normal((1, 4, 6, 6), dtype=np.float32))
    w5 = hip.array(rng.standard_normal((6, 4, 5, 5), dtype=np.float32))
    with pytest.raises(EddlHipError, match="resize first"):
        hip.conv2D(x, w5, None, hip.empty((1, 6, 8, 8)), 1, 1, 0, 0, upsample=(2, 2))
    with pytest.raises(EddlHipError, match="bad upsampling factors"):
        hip.conv2D(x, hip.array(np.zeros((6, 4, 3, 3), np.float32)), None, hip.empty((1, 6, 4, 4)), 1, 1, 0, 0, upsample=(0, 2))


WINOGRAD_CASES = [
    # N, C (all input channels), H, W (stored), Kf, (pad top, pad left), (P, Q) or None, bias, bn, residual, relu, two tensors, upsampling
    (2, 16, 8, 8, 32, (1, 1), None, False, False, False, False, False, None),
    (1, 5, 9, 7, 7, (1, 1), None, True, False, False, True, False, None),            # odd output sizes, ragged channels and filters
    (3, 32, 14, 14, 64, (1, 1), None, False, True, True, True, False, None),         # the whole fused epilogue
    (2, 48, 13, 17, 40, (0, 0), None, True, False, False, False, False, None),       # no padding
    (2, 32, 12, 16, 40, (2, 1), None, False, True, False, False, False, None),       # a folded Pad layer: unequal paddings
    (2, 16, 10, 10, 16, (0, 0), (9, 9), False, False, False, False, False, None),    # zero rows below and right of the image only
    (2, 32, 12, 12, 48, (1, 1), None, False, True, False, True, True, None),         # a folded Concat
    (2, 16, 6, 5, 24, (1, 1), None, True, False, False, False, False, (2, 2)),       # a folded UpSampling2D
    (1, 16, 6, 6, 24, (0, 0), (11, 11), False, False, False, False, False, (2, 3)),
    (4, 256, 28, 28, 256, (1, 1), None, False, True, False, True, False, None),      # a long channel sum
    (2, 24, 11, 20, 40, (0, 0), None, True, False, False, False, False, None),       # rows of a multiple of four pixels: 16-byte pixel loads, no padding
    (2, 16, 12, 24, 24, (1, 2), None, False, False, False, True, False, None),       # the same with two columns of padding
]


WINOGRAD_FORMS = [(4, 1), (5, 1), (6, 1), (7, 1), (6, 4), (7, 3)]
WINOGRAD_FORM_IDS = ["three-kernels", "folded", "one-launch-32x32", "one-launch-64x32", "one-launch-32x32-4-slices", "one-launch-64x32-3-slices"]


@pytest.mark.parametrize("form", WINOGRAD_FORMS, ids=WINOGRAD_FORM_IDS)
@pytest.mark.parametrize("case", WINOGRAD_CASES, ids=lambda c: "x".join(str(v) for v in c[:5]))
def test_conv2d_winograd_form_against_oracle(hip, oracle, case, form):
    """The Winograd forms (force_conv_plan(4, .): transforms and products as separate launches; 5: the output transform
    folded into the one product launch, for channel counts that are whole K-steps; (6, s) and (7, s): everything in one
    launch that reads the input itself, on 32- and 64-filter tiles, the tiles divided into s slices along the channels and
    finished by a second kernel when s > 1) against the CPU oracle's direct convolution of the same logical input
    (concatenated / resized / zero-padded on the host), to the convolution tolerance; the epilogue after it is the
    oracle's, step by step."""
    form, variant = form
    N, C, H, W, Kf, (pt, pl), out, use_bias, use_bn, use_res, relu, two, up = case
    rng = np.random.default_rng(77)
    Ci = C // 2 if two else C
    a = rng.standard_normal((N, Ci, H, W), dtype=np.float32)
    b = rng.standard_normal((N, Ci, H, W), dtype=np.float32) if two else None
    w = (rng.standard_normal((Kf, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    logical = np.concatenate([a, b], axis=1) if two else a
    if up:
        logical = np.repeat(np.repeat(logical, up[0], axis=2), up[1], axis=3)
    Hu, Wu = logical.shape[2:]
    P, Q = out or (Hu + 2 * pt - 2, Wu + 2 * pl - 2)
    # the output size fixes how many zero rows / columns follow the image
    padded = np.zeros((N, C, P + 2, Q + 2), np.float32)
    ys, xs = min(Hu, P + 2 - pt), min(Wu, Q + 2 - pl)
    padded[:, :, pt:pt + ys, pl:pl + xs] = logical[:, :, :ys, :xs]
    bias = rng.standard_normal(Kf, dtype=np.float32) if use_bias else None
    bn = _bn_params(rng, Kf) if use_bn else None
    res = rng.standard_normal((N, Kf, P, Q), dtype=np.float32) if use_res else None
    ref = oracle.conv2d(padded, w, bias, (1, 1), 0, 0, P, Q)
    if bn is not None:
        g, bb, mean, var, eps = bn
        ref, _, _ = oracle.batchnorm_inference(ref, mean, var, g, bb, eps)
    if res is not None:
        ref = oracle.add(ref, res)
    if relu:
        ref = oracle.relu(ref)
    O = hip.full((N, Kf, P, Q), 3.0)
    dbn = (hip.array(bn[0]), hip.array(bn[1]), hip.array(bn[2]), hip.array(bn[3]), bn[4]) if bn else None
    hip.force_conv_plan(form, variant)
    try:
        hip.conv2D(hip.array(a), hip.array(w), hip.array(bias) if use_bias else None, O, 1, 1, pt, pl, bn=dbn,
                   residual=hip.array(res) if use_res else None, relu=relu, second=hip.array(b) if two else None, upsample=up)
        name = hip.last_conv_kernel()
    finally:
        hip.force_conv_plan(-1, 1)
    if form != 5 or C % 16 == 0:
        assert name.startswith("winograd[") and ("true,true>" in name) == (form == 5) and ("wino_fused_kernel" in name) == (form >= 6), name
        assert ("+ksplit" in name) == (form >= 6 and variant > 1 and C > 4), name
    else:
        assert not name.startswith("winograd["), name       # the folded form needs whole K-steps of channels: the direct form ran
    assert_conv_close(ref, O.numpy(), "winograd %s" % (case,))


@pytest.mark.parametrize("form", [4, 5], ids=["three-kernels", "folded"])
def test_conv2d_winograd_form_of_2x2_filters_against_oracle(hip, oracle, form):
    """F(2x2, 2x2): the convolutions behind U-Net's upsamplings (a folded UpSampling2D and a folded Pad of one row below and
    one column right), plain 2x2 'valid' convolutions, odd sizes, the fused epilogue - against the oracle's direct form."""
    rng = np.random.default_rng(79)
    cases = [(2, 32, 8, 8, 48, (0, 0), None, None), (1, 16, 9, 11, 24, (0, 0), None, None), (2, 32, 6, 6, 16, (0, 0), (12, 12), (2, 2)),
             (2, 64, 5, 7, 40, (1, 0), None, None), (1, 48, 7, 5, 32, (0, 0), (14, 10), (2, 2))]
    for (N, C, H, W, Kf, (pt, pl), out, up) in cases:
        a = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, 2, 2)) * np.sqrt(2.0 / (C * 4))).astype(np.float32)
        logical = np.repeat(np.repeat(a, up[0], axis=2), up[1], axis=3) if up else a
        Hu, Wu = logical.shape[2:]
        P, Q = out or (Hu + 2 * pt - 1, Wu + 2 * pl - 1)
        padded = np.zeros((N, C, P + 1, Q + 1), np.float32)
        ys, xs = min(Hu, P + 1 - pt), min(Wu, Q + 1 - pl)
        padded[:, :, pt:pt + ys, pl:pl + xs] = logical[:, :, :ys, :xs]
        bias = rng.standard_normal(Kf, dtype=np.float32)
        bn = _bn_params(rng, Kf)
        ref = oracle.conv2d(padded, w, bias, (1, 1), 0, 0, P, Q)
        ref, _, _ = oracle.batchnorm_inference(ref, bn[2], bn[3], bn[0], bn[1], bn[4])
        ref = oracle.relu(ref)
        O = hip.full((N, Kf, P, Q), 3.0)
        dbn = (hip.array(bn[0]), hip.array(bn[1]), hip.array(bn[2]), hip.array(bn[3]), bn[4])
        hip.force_conv_plan(form, 1)
        try:
            hip.conv2D(hip.array(a), hip.array(w), hip.array(bias), O, 1, 1, pt, pl, bn=dbn, relu=True, upsample=up)
            name = hip.last_conv_kernel()
        finally:
            hip.force_conv_plan(-1, 1)
        assert name.startswith("winograd[") and ("true,true>" in name) == (form == 5), name
        assert_conv_close(ref, O.numpy(), "winograd 2x2 %s" % ((N, C, H, W, Kf, pt, pl, out, up),))


UP2X2_FORM = 8      # force_conv_plan tiles 8 and 9: the upsampled-input form of a 2x2 filter


def test_conv2d_upsampled_2x2_form_against_oracle(hip, oracle):
    """A 2x2 filter on an input upsampled twice, run as four convolutions of the stored image (one per parity of the output
    row and column, weight sums as filters: force_conv_plan(8, .) / (9, .)): U-Net's decoder step (UpSampling2D, Pad of one row below
    and one column right, Conv 2x2) in small, 'valid' and over-padded output sizes, odd stored sizes, ragged filter counts,
    channel counts that are whole K-steps of four, the fused epilogue with and without a residual - against the oracle's direct convolution of
    the upsampled, padded tensor; with registered filters (the nine matrices kept, following a write); with the 2x2 max-pool
    in its epilogue bit for bit the pool kernel's; and where the form does not apply the planner's plan runs."""
    rng = np.random.default_rng(88)
    # N, C, H, W (stored), Kf, output size or None (2H x 2W: one row / column of zeros), residual
    cases = [(2, 32, 6, 6, 16, None, False), (1, 44, 7, 5, 33, None, True), (3, 12, 5, 9, 70, (9, 17), False), (2, 64, 4, 4, 64, (9, 10), True),
             (1, 96, 11, 3, 24, (21, 5), False), (5, 32, 8, 8, 128, None, False), (1, 8, 5, 5, 32, None, False), (2, 4, 6, 7, 16, None, True)]
    for (N, C, H, W, Kf, out, use_res) in cases:
        a = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, 2, 2)) * np.sqrt(2.0 / (C * 4))).astype(np.float32)
        logical = np.repeat(np.repeat(a, 2, axis=2), 2, axis=3)
        P, Q = out or (2 * H, 2 * W)
        padded = np.zeros((N, C, P + 1, Q + 1), np.float32)
        ys, xs = min(2 * H, P + 1), min(2 * W, Q + 1)
        padded[:, :, :ys, :xs] = logical[:, :, :ys, :xs]
        bias = rng.standard_normal(Kf, dtype=np.float32)
        bn = _bn_params(rng, Kf)
        res = rng.standard_normal((N, Kf, P, Q), dtype=np.float32) if use_res else None
        ref = oracle.conv2d(padded, w, bias, (1, 1), 0, 0, P, Q)
        ref, _, _ = oracle.batchnorm_inference(ref, bn[2], bn[3], bn[0], bn[1], bn[4])
        if use_res:
            ref = ref + res
        ref = oracle.relu(ref)
        O = hip.full((N, Kf, P, Q), 3.0)
        dbn = (hip.array(bn[0]), hip.array(bn[1]), hip.array(bn[2]), hip.array(bn[3]), bn[4])
        form = UP2X2_FORM + (N % 2)                 # (the kernel built for three workgroups per CU, or for two)
        hip.force_conv_plan(form, 1)
        try:
            hip.conv2D(hip.array(a), hip.array(w), hip.array(bias), O, 1, 1, 0, 0, bn=dbn, residual=hip.array(res) if use_res else None, relu=True,
                       upsample=(2, 2))
            name = hip.last_conv_kernel()
        finally:
            hip.force_conv_plan(-1, 1)
        assert name.startswith("upsampled2x2[conv_up2x2_kernel<%d>," % (3 if form == UP2X2_FORM else 2)), name
        assert_conv_close(ref, O.numpy(), "upsampled 2x2 %s" % ((N, C, H, W, Kf, out, use_res),))

    # the two builds of the kernel (three and two workgroups per CU; row-by-row and four-row epilogue) sum in one order
    for (N, C, H, W, Kf) in ((3, 40, 9, 7, 70), (2, 128, 16, 16, 64)):
        a = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, 2, 2)) * 0.1).astype(np.float32)
        bn = _bn_params(rng, Kf)
        dbn = (hip.array(bn[0]), hip.array(bn[1]), hip.array(bn[2]), hip.array(bn[3]), bn[4])
        outs = []
        for form in (UP2X2_FORM, UP2X2_FORM + 1):
            O = hip.full((N, Kf, 2 * H, 2 * W), float(form))
            hip.force_conv_plan(form, 1)
            try:
                hip.conv2D(hip.array(a), hip.array(w), None, O, 1, 1, 0, 0, bn=dbn, relu=True, upsample=(2, 2))
            finally:
                hip.force_conv_plan(-1, 1)
            outs.append(O.numpy())
        assert np.array_equal(outs[0], outs[1]), (N, C, H, W, Kf)

    # registered filters: the nine matrices are kept and follow a write; the pool in the epilogue
    N, C, H, W, Kf = 2, 32, 6, 8, 40
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 2, 2)) * 0.1).astype(np.float32)
    X, Wd = hip.array(x), hip.array(w)
    O1, O2, O3 = (hip.full((N, Kf, 2 * H, 2 * W), v) for v in (1.0, 2.0, 3.0))
    pooled = lambda: tuple(hip.full((N, Kf, H, W), 7.0) for _ in range(3))
    A, B = pooled(), pooled()
    hip.cache_conv_filters(Wd)
    hip.force_conv_plan(UP2X2_FORM, 1)
    try:
        hip.conv2D(X, Wd, None, O1, 1, 1, 0, 0, upsample=(2, 2))
        assert hip.last_conv_kernel().startswith("upsampled2x2[")
        first = O1.numpy()
        up = np.repeat(np.repeat(x, 2, axis=2), 2, axis=3)
        padded = np.zeros((N, C, 2 * H + 1, 2 * W + 1), np.float32)
        padded[:, :, :2 * H, :2 * W] = up
        assert_conv_close(oracle.conv2d(padded, w, None, (1, 1), 0, 0, 2 * H, 2 * W), first, "kept filters")
        Wd.copy_from(2.0 * w)
        hip.conv2D(X, Wd, None, O2, 1, 1, 0, 0, upsample=(2, 2))
        assert np.array_equal(O2.numpy(), 2.0 * first)          # doubling is exact in the weight sums and in every product
        hip.mpool2D(O2, A[0], A[1], A[2], (2, 2), (2, 2), (0, 0, 0, 0))
        hip.conv2D(X, Wd, None, O3, 1, 1, 0, 0, upsample=(2, 2), pool=B, keep=True)
        assert hip.last_conv_kernel().startswith("upsampled2x2[") and np.array_equal(O3.numpy(), O2.numpy())
        for u, v, what in zip(A, B, ("pooled", "indX", "indY")):
            assert np.array_equal(u.numpy(), v.numpy()), what
        # where it does not apply (a stored tensor, a padding above / left, a channel count that is no whole K-step): the planner's plan
        hip.conv2D(hip.array(up), Wd, None, O1, 1, 1, 0, 0)
        assert not hip.last_conv_kernel().startswith("upsampled2x2[")
        O4 = hip.empty((N, Kf, 2 * H + 1, 2 * W + 1))
        hip.conv2D(X, Wd, None, O4, 1, 1, 1, 1, upsample=(2, 2))
        assert not hip.last_conv_kernel().startswith("upsampled2x2[")
        w22 = hip.array((rng.standard_normal((Kf, 22, 2, 2)) * 0.1).astype(np.float32))
        hip.conv2D(hip.array(x[:, :22].copy()), w22, None, O1, 1, 1, 0, 0, upsample=(2, 2))
        assert not hip.last_conv_kernel().startswith("upsampled2x2[")
    finally:
        hip.force_conv_plan(-1, 1)
        hip.uncache_conv_filters(Wd)


def _misaligned_copy(hip, host):
    """A device copy of `host` that starts four bytes into its allocation, i.e. not at a multiple of 16 bytes."""
    from eddl_amd.backend import _View
    base = hip.empty((host.size + 1,))
    full = np.zeros(host.size + 1, np.float32)
    full[1:] = host.ravel()
    base.copy_from(full)
    view = object.__new__(_View)
    view.backend, view.ptr, view.size, view.nbytes, view.shape, view._base = hip, base.ptr + 4, host.size, host.size * 4, host.shape, base
    return view


@pytest.mark.parametrize("form", [(6, 1), (7, 1), (7, 3)], ids=["32x32", "64x32", "64x32-3-slices"])
def test_conv2d_one_launch_pixel_loads_of_16_and_of_4_bytes_give_the_same_bits(hip, form):
    """The one-launch Winograd kernel loads the pixels 16 bytes per lane where image rows are a multiple of four pixels
    and the tensors are 16-byte aligned, 4 bytes per lane otherwise: the same input at an address that is not a multiple
    of 16 takes the other build and gives the same output bit for bit (one and two input tensors, with and without
    padding, rows of blocks that end inside a tile)."""
    rng = np.random.default_rng(91)
    cases = [(3, 24, 16, 24, 40, (1, 1), False), (2, 32, 11, 20, 70, (0, 0), False), (2, 32, 12, 12, 48, (1, 1), True),
             (2, 16, 12, 24, 24, (1, 2), False), (5, 64, 28, 28, 64, (1, 1), False)]
    for _ in range(12):  # and random ones: rows of 12 ... 64 pixels, any height, ragged channel and filter counts
        two = bool(rng.integers(0, 2))
        cases.append((int(rng.integers(1, 5)), int(rng.integers(2, 36)) * (2 if two else 1), int(rng.integers(5, 40)), 4 * int(rng.integers(3, 17)),
                      int(rng.integers(8, 140)), (int(rng.integers(0, 3)), int(rng.integers(0, 3))), two))
    for N, C, H, W, Kf, (pt, pl), two in cases:
        Ci = C // 2 if two else C
        a = rng.standard_normal((N, Ci, H, W), dtype=np.float32)
        b = rng.standard_normal((N, Ci, H, W), dtype=np.float32) if two else None
        w = hip.array((rng.standard_normal((Kf, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32))
        P, Q = H + 2 * pt - 2, W + 2 * pl - 2
        outs = []
        for misaligned in (False, True):
            da = _misaligned_copy(hip, a) if misaligned else hip.array(a)
            db = None if not two else (_misaligned_copy(hip, b) if misaligned else hip.array(b))
            assert (da.ptr % 16 != 0) == misaligned
            O = hip.full((N, Kf, P, Q), 3.0)
            hip.force_conv_plan(*form)
            try:
                hip.conv2D(da, w, None, O, 1, 1, pt, pl, relu=True, second=db)
                name = hip.last_conv_kernel()
                # (the 16-byte build where it applies - rows of at least six blocks - and only at an aligned address)
                assert "wino_fused_kernel" in name and (",true>" in name) == (not misaligned and (Q + 1) // 2 >= 6), name
            finally:
                hip.force_conv_plan(-1, 1)
            outs.append(O.numpy())
        assert np.array_equal(outs[0], outs[1]), (N, C, H, W, Kf, pt, pl, two)


def test_conv2d_winograd_form_only_where_it_applies_and_with_kept_filters(hip, oracle):
    """Strides other than one and filters other than 3x3 keep the direct form under force_conv_plan(4, .) and set_conv_algo
    ("winograd"); registered filters keep their transformed copy, which follows writes to the filter tensor; the call that
    cannot allocate never takes the Winograd form."""
    rng = np.random.default_rng(78)
    x = rng.standard_normal((2, 16, 12, 12), dtype=np.float32)
    w3 = (rng.standard_normal((32, 16, 3, 3)) * 0.1).astype(np.float32)
    w1 = (rng.standard_normal((32, 16, 1, 1)) * 0.1).astype(np.float32)
    hip.set_conv_algo("winograd")
    try:
        ref, out = run_conv(hip, oracle, x, w3, None, (2, 2), "same", algo=7)
        assert not hip.last_conv_kernel().startswith("winograd") and (assert_conv_close(ref, out, "stride 2") is None)
        ref, out = run_conv(hip, oracle, x, w1, None, (1, 1), "valid", algo=7)
        assert not hip.last_conv_kernel().startswith("winograd") and (assert_conv_close(ref, out, "1x1") is None)
        ref, out = run_conv(hip, oracle, x, w3, None, (1, 1), "same", algo=7)
        assert hip.last_conv_kernel().startswith("winograd") and (assert_conv_close(ref, out, "3x3") is None)
        # kept filters: the transformed copy is made on first use and redone after a write
        X, Wd, O = hip.array(x), hip.array(w3), hip.empty((2, 32, 12, 12))
        hip.cache_conv_filters(Wd)
        hip.set_conv_algo(7)
        hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)
        assert hip.last_conv_kernel().startswith("winograd")
        first = O.numpy()
        assert_conv_close(oracle.conv2d(x, w3, None, (1, 1), 1, 1, 12, 12), first, "kept filters")
        Wd.copy_from(2.0 * w3)
        hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)
        assert np.array_equal(O.numpy(), 2.0 * first)      # doubling is exact in every step of the transforms
        # the entry point over the fixed scratch array keeps the direct form
        O2, O3 = hip.empty((2, 32, 12, 12)), hip.empty((2, 32, 12, 12))
        hip._check(hip.lib.eddlhip_conv2d_fwd_noalloc(hip.dev, X.ptr, Wd.ptr, None, O2.ptr, 2, 16, 12, 12, 32, 3, 3, 1, 1, 1, 1, 12, 12,
                                                      None, None, None, None, 0.0, None, 0))
        assert not hip.last_conv_kernel().startswith("winograd")
        hip.set_conv_algo("winograd_off")
        hip.conv2D(X, Wd, None, O3, 1, 1, 1, 1)
        assert np.array_equal(O2.numpy(), O3.numpy())
        hip.uncache_conv_filters(Wd)
    finally:
        hip.set_conv_algo("winograd_off")
        hip.set_conv_algo("auto")


@pytest.mark.parametrize("form", [-1, 4, 5, 6, 7, 9])
@pytest.mark.parametrize("case", ["bias+relu", "bn+residual+relu", "2x2 filter", "two tensors", "upsampled", "nan window"])
def test_conv2d_fwd_maxpool_is_the_convolution_followed_by_the_pool(hip, form, case):
    """eddlhip_conv2d_fwd_maxpool against eddlhip_conv2d_fwd* + eddlhip_maxpool2d(2, 2, 2, 2) under the same launch plan
    (the planner's direct form, the Winograd form in three kernels, the folded Winograd form): pooled values and both
    index tensors bit for bit, the unpooled output too when it is kept; a window of NaN leaves the indices as they were."""
    cases = ["bias+relu", "bn+residual+relu", "2x2 filter", "two tensors", "upsampled", "nan window"]
    rng = np.random.default_rng(500 + 10 * (form + 1) + cases.index(case))
    N, C, H, W, Kf, fs = 3, 32, 12, 16, 48, 3
    second = upsample = None
    if case == "2x2 filter":
        fs = 2
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    X = hip.array(x)
    if case == "two tensors":
        second = hip.array(rng.standard_normal((N, C, H, W), dtype=np.float32))
    if case == "upsampled":
        upsample = (2, 2)
    Cin = 2 * C if second is not None else C
    Hu, Wu = (H * 2, W * 2) if upsample else (H, W)
    w = hip.array((rng.standard_normal((Kf, Cin, fs, fs)) * 0.1).astype(np.float32))
    pad = 1 if fs == 3 else 0
    P, Q = (Hu, Wu) if fs == 3 else (Hu, Wu)          # 2x2: one more row and column of zeros below and to the right
    bias = hip.array(rng.standard_normal(Kf).astype(np.float32)) if case in ("bias+relu", "2x2 filter", "nan window") else None
    bn = res = None
    if case == "bn+residual+relu":
        bn = (hip.array(rng.uniform(0.8, 1.2, Kf).astype(np.float32)), hip.array((rng.standard_normal(Kf) * 0.1).astype(np.float32)),
              hip.array((rng.standard_normal(Kf) * 0.1).astype(np.float32)), hip.array(rng.uniform(0.5, 1.5, Kf).astype(np.float32)), 1e-5)
    if case in ("bn+residual+relu", "nan window"):
        r = rng.standard_normal((N, Kf, P, Q), dtype=np.float32)
        if case == "nan window":
            r[1, 5, 4:6, 6:8] = np.nan
        res = hip.array(r)
    relu = case != "nan window"                        # (the ReLU of this path turns NaN into 0)
    O1, O2 = hip.full((N, Kf, P, Q), 3.0), hip.full((N, Kf, P, Q), 4.0)
    pooled = lambda: (hip.full((N, Kf, P // 2, Q // 2), 9.0), hip.full((N, Kf, P // 2, Q // 2), 7.0), hip.full((N, Kf, P // 2, Q // 2), 7.0))
    A, B, K2 = pooled(), pooled(), pooled()
    variant = 1
    if form == 9:                                      # the one-launch form on its 64-filter tile, three K slices per tile
        form, variant = 7, 3
    try:
        hip.force_conv_plan(form, variant)
        hip.conv2D(X, w, bias, O1, 1, 1, pad, pad, bn=bn, residual=res, relu=relu, second=second, upsample=upsample)
        name = hip.last_conv_kernel()
        assert name.startswith("winograd") == (form >= 4 and not (form >= 6 and fs == 2)), name   # (the one-launch form: 3x3 filters only)
        hip.mpool2D(O1, A[0], A[1], A[2], (2, 2), (2, 2), (0, 0, 0, 0))
        hip.conv2D(X, w, bias, O2, 1, 1, pad, pad, bn=bn, residual=res, relu=relu, second=second, upsample=upsample, pool=B, keep=True)
        assert hip.last_conv_kernel() == name
        ref = O1.numpy()
        assert np.array_equal(ref, O2.numpy(), equal_nan=True), name
        for a, b, what in zip(A, B, ("pooled", "indX", "indY")):
            assert np.array_equal(a.numpy(), b.numpy()), what + " " + name
        if case == "nan window":
            assert A[0].numpy()[1, 5, 2, 3] == np.float32(-3.40282e38) and A[1].numpy()[1, 5, 2, 3] == 7.0
        # without the unpooled output: the same pooled tensors; a Winograd form leaves O alone
        O3 = hip.full((N, Kf, P, Q), 5.0)
        hip.conv2D(X, w, bias, O3, 1, 1, pad, pad, bn=bn, residual=res, relu=relu, second=second, upsample=upsample, pool=K2, keep=False)
        for a, b, what in zip(A, K2, ("pooled", "indX", "indY")):
            assert np.array_equal(a.numpy(), b.numpy()), what + " without the output, " + name
        if name.startswith("winograd"):
            assert np.all(O3.numpy() == 5.0)
        # the gathered maxima are the kept outputs at the reported coordinates
        if case != "nan window":
            n, k = np.indices(A[0].shape)[:2]
            assert np.array_equal(ref[n, k, A[2].numpy().astype(np.int64), A[1].numpy().astype(np.int64)], A[0].numpy())
    finally:
        hip.force_conv_plan(-1, 1)


def test_conv2d_fwd_maxpool_refuses_odd_output_planes(hip):
    X, w, O = hip.array(np.zeros((1, 4, 7, 8), np.float32)), hip.array(np.zeros((8, 4, 3, 3), np.float32)), hip.empty((1, 8, 7, 8))
    pooled = (hip.empty((1, 8, 3, 4)), hip.empty((1, 8, 3, 4)), hip.empty((1, 8, 3, 4)))
    with pytest.raises(Exception, match="even sides"):
        hip.conv2D(X, w, None, O, 1, 1, 1, 1, pool=pooled)


def test_conv2d_winograd_never_keeps_infinities_where_the_direct_form_has_them(hip):
    """set_conv_algo("winograd_never"): neither a forced plan nor the plan search takes a Winograd form, so an infinity in
    the input stays an infinity in exactly the outputs whose window holds it (the transforms would subtract it from itself)."""
    rng = np.random.default_rng(91)
    x = rng.standard_normal((4, 64, 28, 28), dtype=np.float32)
    x[1, 3, 5, 7] = np.inf
    w = (rng.standard_normal((64, 64, 3, 3)) * 0.05).astype(np.float32)
    X, Wd, O = hip.array(x), hip.array(w), hip.empty((4, 64, 28, 28))
    hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)
    direct = O.numpy()
    window = np.zeros((4, 64, 28, 28), bool)
    window[1, :, 4:7, 6:9] = True
    assert np.array_equal(np.isinf(direct), window) and not np.isnan(direct).any()
    hip.conv_autotune(-1)
    try:
        hip.set_conv_algo("winograd_never")
        hip.force_conv_plan(4, 1)
        hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)
        assert not hip.last_conv_kernel().startswith("winograd")
        hip.force_conv_plan(-1, 1)
        hip.conv_autotune(True)
        hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)      # searched, without the Winograd candidates
        assert hip.conv_tuned_plans() == 1 and not hip.last_conv_kernel().startswith("winograd")
        got = O.numpy()
        assert np.array_equal(np.isinf(got), window) and not np.isnan(got).any()
        finite = ~window
        assert np.allclose(got[finite], direct[finite], rtol=1e-4, atol=1e-5)
        hip.set_conv_algo("winograd_off")            # back to the default: a forced Winograd plan applies again
        hip.force_conv_plan(4, 1)
        hip.conv2D(X, Wd, None, O, 1, 1, 1, 1)
        assert hip.last_conv_kernel().startswith("winograd")
    finally:
        hip.force_conv_plan(-1, 1)
        hip.set_conv_algo("winograd_off")
        hip.conv_autotune(-1)


def test_conv2d_linearity_and_empty_batch(hip, oracle):
    from eddl_amd.descriptors import ConvolDescriptor
    rng = np.random.default_rng(301)
    x1 = rng.standard_normal((2, 16, 20, 20), dtype=np.float32)
    x2 = rng.standard_normal((2, 16, 20, 20), dtype=np.float32)
    w = rng.standard_normal((32, 16, 3, 3), dtype=np.float32) / 12
    _, o1 = run_conv(hip, oracle, x1, w, None, (1, 1), "same", algo="mfma")
    _, o2 = run_conv(hip, oracle, x2, w, None, (1, 1), "same", algo="mfma")
    _, o12 = run_conv(hip, oracle, x1 + x2, w, None, (1, 1), "same", algo="mfma")
    np.testing.assert_allclose(o12, o1 + o2, rtol=1e-4, atol=1e-4)
    # empty batch: nothing launched, no error
    cd = ConvolDescriptor(32, [3, 3], [1, 1], "same").build([0, 16, 20, 20])
    hip.conv2D(hip.empty((0, 16, 20, 20)), hip.array(w), None, hip.empty(cd.out_shape), 1, 1, 1, 1)
    hip.synchronize()


def test_conv2d_argument_errors(hip):
    from eddl_amd import EddlHipError
    x, w, o = hip.empty((1, 3, 8, 8)), hip.empty((4, 3, 3, 3)), hip.empty((1, 4, 8, 8))
    g = hip.empty((4,))
    with pytest.raises(EddlHipError, match="bn_mean and bn_var"):
        hip.conv2D(x, w, None, o, 1, 1, 1, 1, bn=(None, None, g, None, 1e-5))
    with pytest.raises(EddlHipError, match="strides"):
        hip.conv2D(x, w, None, o, 0, 1, 1, 1)


# ------------------------------------------------------------------ bandwidth-bound operators
def test_batchnorm_inference_bit_exact(hip, oracle):
    rng = np.random.default_rng(400)
    # planes of 16 .. 4095 elements and a multiple of four take the channel-per-workgroup kernel (image groups, partly
    # filled thread rows), other planes below 4096 elements the flat kernel (float4 groups that cross plane borders, a
    # ragged end), larger ones and planes of fewer than 4 elements the plane-per-workgroup kernel
    for shape in [(4, 64, 28, 28), (3, 5, 7, 9), (2, 130, 1, 1), (2, 3, 6, 6), (1, 20000, 1, 2), (2, 7, 5, 1), (2, 70, 7, 7),
                  (1, 3, 7, 7), (1, 2, 64, 63), (1, 2, 64, 64), (3, 2, 70, 70), (5, 300, 2, 2),
                  (70, 3, 14, 14), (9, 33, 56, 56), (2, 2100, 4, 4), (37, 40, 20, 3), (1, 1, 4, 4)]:
        C = shape[1]
        x = rng.standard_normal(shape, dtype=np.float32)
        g, b, mean, var, eps = _bn_params(rng, C)
        y_ref, opa_ref, sd_ref = oracle.batchnorm_inference(x, mean, var, g, b, eps)
        y, opa, sd = hip.empty(shape), hip.empty(shape), hip.empty((C,))
        hip.batchnorm_inference(hip.array(x), y, opa, hip.array(mean), hip.array(var), hip.array(g), hip.array(b), sd, eps)
        assert np.array_equal(y.numpy(), y_ref) and np.array_equal(opa.numpy(), opa_ref) and np.array_equal(sd.numpy(), sd_ref)
        y2_ref, _, _ = oracle.batchnorm_inference(x, mean, var, None, None, eps)
        hip.batchnorm_inference(hip.array(x), y, None, hip.array(mean), hip.array(var), None, None, sd, eps)
        assert np.array_equal(y.numpy(), y2_ref)


def test_relu_add_inc_fill(hip, oracle):
    rng = np.random.default_rng(401)
    for n in (1, 3, 1023, 4096, 100003):
        x = rng.standard_normal(n, dtype=np.float32)
        y = rng.standard_normal(n, dtype=np.float32)
        x[:: 7] = 0.0
        if n > 8:
            x[1], x[2], x[3], x[4] = -0.0, np.nan, np.inf, -np.inf
        B = hip.empty((n,))
        hip.relu(hip.array(x), B)
        out = B.numpy()
        assert np.array_equal(out, oracle.relu(x)) and not np.any(np.signbit(out))
        C = hip.empty((n,))
        x = np.nan_to_num(x, nan=1.0, posinf=2.0, neginf=-2.0)
        hip.add(1.0, hip.array(x), 1.0, hip.array(y), C, 0)
        assert np.array_equal(C.numpy(), oracle.add(x, y))
        hip.add(0.5, hip.array(x), -3.0, hip.array(y), C, 1)
        assert np.array_equal(C.numpy(), oracle.add(x, y, 0.5, -3.0, c=oracle.add(x, y)))
        # the n-ary Add layer: fill_(0) then inc per parent
        hip.fill_(C, 0.0)
        hip.inc(hip.array(x), C)
        hip.inc(hip.array(y), C)
        assert np.array_equal(C.numpy(), (np.float32(0) + x) + y)
        hip.fill_(C, 2.5)
        assert np.all(C.numpy() == np.float32(2.5))


def test_maxpool_bit_exact_with_indices(hip, oracle):
    rng = np.random.default_rng(402)
    cases = [
        ((4, 16, 56, 56), (2, 2), (2, 2), (0, 0, 0, 0)),   # fast path
        ((2, 3, 57, 55), (2, 2), (2, 2), (0, 0, 0, 0)),    # odd sizes: general path
        ((2, 8, 28, 28), (3, 3), (2, 2), (1, 1, 1, 1)),    # ResNet stem pool geometry
        ((2, 4, 13, 17), (3, 3), (1, 1), (1, 1, 1, 1)),
        # 3x3 stride 2, two outputs per thread: left pad 1 and 0, rows that end inside a wavefront, a ragged last wavefront
        ((2, 3, 112, 112), (3, 3), (2, 2), (1, 1, 1, 1)),
        ((2, 4, 28, 28), (3, 3), (2, 2), (0, 1, 0, 1)),
        ((2, 2, 30, 32), (3, 3), (2, 2), (0, 1, 1, 0)),
        ((1, 2, 12, 264), (3, 3), (2, 2), (1, 1, 1, 1)),
        ((1, 2, 11, 264), (3, 3), (2, 2), (2, 0, 0, 1)),
        ((1, 1, 8, 12), (3, 3), (2, 2), (1, 1, 1, 1)),
        ((1, 3, 20, 22), (3, 3), (2, 2), (1, 1, 1, 1)),    # width not a multiple of 4: one output per thread
        ((2, 4, 12, 12), (2, 2), (2, 2), (0, 1, 0, 1)),
        ((3, 5, 7, 7), (7, 7), (1, 1), (0, 0, 0, 0)),      # 49 taps, one thread per output
        ((3, 5, 9, 9), (9, 9), (1, 1), (0, 0, 0, 0)),      # 81 taps: one wavefront per output
        ((2, 3, 20, 20), (8, 8), (4, 4), (2, 2, 2, 2)),    # wavefront path with padding
    ]
    for shape, k, s, pads in cases:
        for ties in (False, True):
            x = rng.integers(-3, 4, size=shape).astype(np.float32) if ties else rng.standard_normal(shape, dtype=np.float32)
            O_ref, ix_ref, iy_ref = oracle.maxpool2d(x, k, s, pads, fill=-5.0)
            O, ix, iy = hip.empty(O_ref.shape), hip.full(O_ref.shape, -5.0), hip.full(O_ref.shape, -5.0)
            assert hip.pool_out_dims(shape[2], shape[3], k, s, pads) == O_ref.shape[2:]
            hip.mpool2D(hip.array(x), O, ix, iy, k, s, pads)
            assert np.array_equal(O.numpy(), O_ref), (shape, k)
            assert np.array_equal(ix.numpy(), ix_ref) and np.array_equal(iy.numpy(), iy_ref), (shape, k, ties)
    # windows with nothing above the start value keep their index slots
    for shape, k in (((1, 2, 8, 8), (2, 2)), ((1, 2, 9, 9), (3, 3)), ((1, 1, 16, 16), (8, 8))):
        x = np.full(shape, -np.inf, np.float32)
        x[0, 0, :4, :4] = np.nan
        O_ref, ix_ref, iy_ref = oracle.maxpool2d(x, k, k, (0, 0, 0, 0), fill=-5.0)
        O, ix, iy = hip.empty(O_ref.shape), hip.full(O_ref.shape, -5.0), hip.full(O_ref.shape, -5.0)
        hip.mpool2D(hip.array(x), O, ix, iy, k, k, (0, 0, 0, 0))
        assert np.array_equal(O.numpy(), O_ref) and np.array_equal(ix.numpy(), ix_ref) and np.array_equal(iy.numpy(), iy_ref)
    for pads in ((1, 1, 1, 1), (0, 1, 0, 1)):  # the same through the 3x3 stride-2 kernel, half of the plane finite
        x = np.full((1, 2, 16, 16), -np.inf, np.float32)
        x[0, 0, :4, :4] = np.nan
        x[0, 1, 8:, :] = rng.standard_normal((8, 16), dtype=np.float32)
        O_ref, ix_ref, iy_ref = oracle.maxpool2d(x, (3, 3), (2, 2), pads, fill=-5.0)
        O, ix, iy = hip.empty(O_ref.shape), hip.full(O_ref.shape, -5.0), hip.full(O_ref.shape, -5.0)
        hip.mpool2D(hip.array(x), O, ix, iy, (3, 3), (2, 2), pads)
        assert np.array_equal(O.numpy(), O_ref) and np.array_equal(ix.numpy(), ix_ref) and np.array_equal(iy.numpy(), iy_ref)


def test_avgpool_bit_exact(hip, oracle):
    rng = np.random.default_rng(403)
    for shape, k, s, pads in [((4, 16, 56, 56), (2, 2), (2, 2), (0, 0, 0, 0)), ((2, 8, 28, 28), (3, 3), (2, 2), (1, 1, 1, 1)),
                              ((2, 64, 7, 7), (7, 7), (1, 1), (0, 0, 0, 0)), ((2, 4, 13, 17), (3, 2), (1, 2), (1, 0, 0, 1)),
                              # whole-plane windows (global average pool): ragged plane counts, even and odd plane sizes,
                              # the largest plane of the LDS kernel and one beyond it
                              ((3, 67, 7, 7), (7, 7), (1, 1), (0, 0, 0, 0)), ((1, 5, 8, 8), (8, 8), (1, 1), (0, 0, 0, 0)),
                              ((2, 130, 15, 17), (15, 17), (1, 1), (0, 0, 0, 0)), ((2, 9, 16, 16), (16, 16), (1, 1), (0, 0, 0, 0)),
                              ((1, 3, 1, 1), (1, 1), (1, 1), (0, 0, 0, 0))]:
        x = rng.standard_normal(shape, dtype=np.float32)
        ref = oracle.avgpool2d(x, k, s, pads)
        O = hip.empty(ref.shape)
        hip.avgpool2D(hip.array(x), O, k, s, pads)
        assert np.array_equal(O.numpy(), ref), (shape, k)


def test_upsample_concat_pad_bit_exact(hip, oracle):
    from eddl_amd import EddlHipError
    rng = np.random.default_rng(404)
    x = rng.standard_normal((2, 5, 9, 7), dtype=np.float32)
    for s in (2, 3):
        ref = oracle.scale_nearest(x, (9 * s, 7 * s))
        B = hip.empty(ref.shape)
        hip.scale(hip.array(x), B, (9 * s, 7 * s))
        assert np.array_equal(B.numpy(), ref)
    for shape in [(3, 4, 10, 12), (1, 2, 1, 2), (2, 3, 33, 64), (1, 1, 512, 510)]:  # exact doubling, even width: the float4 path
        y = rng.standard_normal(shape, dtype=np.float32)
        ref = oracle.scale_nearest(y, (shape[2] * 2, shape[3] * 2))
        B = hip.empty(ref.shape)
        hip.scale(hip.array(y), B, (shape[2] * 2, shape[3] * 2))
        assert np.array_equal(B.numpy(), ref), shape
    ref = oracle.scale_nearest(x, (13, 10))  # non-integer factor, same float rule
    B = hip.empty(ref.shape)
    hip.scale(hip.array(x), B, (13, 10))
    assert np.array_equal(B.numpy(), ref)
    with pytest.raises(EddlHipError, match="outside the source"):
        hip.scale(hip.array(x), hip.empty((2, 5, 18, 14)), (9, 7))  # zoom-out window: no nearest rule
    parts = [rng.standard_normal((2, c, 8, 8), dtype=np.float32) for c in (4, 3, 9)]
    for axis in (1, 0, 3):
        ps = parts if axis == 1 else [parts[0], parts[0] * 2]
        ref = oracle.concat(ps, axis)
        out = hip.empty(ref.shape)
        hip.concat(out, [hip.array(p) for p in ps], axis)
        assert np.array_equal(out.numpy(), ref), axis
    odd = [rng.standard_normal((2, c, 5, 3), dtype=np.float32) for c in (1, 2)]  # scalar path
    out = hip.empty((2, 3, 5, 3))
    hip.concat(out, [hip.array(p) for p in odd], 1)
    assert np.array_equal(out.numpy(), np.concatenate(odd, 1))
    ref = oracle.pad(x, (0, 1, 1, 0), cval=0.0)
    B = hip.full(ref.shape, 0.0)
    hip.pad(hip.array(x), B, (0, 1, 1, 0))
    assert np.array_equal(B.numpy(), ref)
    ref = oracle.pad(x, (1, 2, 3, 4), cval=7.0)
    B = hip.full(ref.shape, 7.0)
    hip.pad(hip.array(x), B, (1, 2, 3, 4))
    assert np.array_equal(B.numpy(), ref)
    # rows of 64 pixels and more take the row-per-wavefront kernel: widths around its 256-pixel step and 64-pixel remainder
    for shape, pads in [((2, 3, 5, 64), (0, 1, 1, 0)), ((1, 2, 7, 65), (2, 0, 0, 3)), ((1, 3, 4, 255), (1, 1, 1, 1)),
                        ((2, 1, 3, 256), (0, 1, 1, 0)), ((1, 2, 6, 449), (3, 2, 1, 5)), ((1, 1, 9, 1030), (0, 0, 0, 1)),
                        ((1, 5, 1100, 70), (1, 0, 0, 0))]:
        y = rng.standard_normal(shape, dtype=np.float32)
        ref = oracle.pad(y, pads, cval=-2.0)
        B = hip.full(ref.shape, -2.0)
        hip.pad(hip.array(y), B, pads)
        assert np.array_equal(B.numpy(), ref), (shape, pads)


def test_dense_sigmoid_softmax_within_tolerance(hip, oracle):
    rng = np.random.default_rng(405)
    for m, k, n in [(32, 512, 1000), (5, 37, 300), (64, 2048, 10), (33, 100, 65), (70, 1001, 131), (32, 3136, 4096), (1, 2, 1),
                    (128, 777, 256), (129, 300, 132), (200, 64, 40), (96, 2048, 1000)]:  # 4, 5, 7, 3 row tiles: one pass over the weights serves four
        a = rng.standard_normal((m, k), dtype=np.float32)
        w = (rng.standard_normal((k, n)) * np.sqrt(2.0 / k)).astype(np.float32)
        bias = rng.standard_normal(n, dtype=np.float32)
        ref = oracle.dense(a, w, bias)
        C = hip.empty((m, n))
        hip.mult2D(hip.array(a), hip.array(w), C)
        hip.sum2D_rowwise(C, hip.array(bias), C)
        assert_conv_close(ref, C.numpy(), "dense %dx%dx%d" % (m, k, n))
        # the one-call form equals mult2D + sum2D_rowwise (+ ReLU) bit for bit
        F = hip.empty((m, n))
        hip.dense(hip.array(a), hip.array(w), hip.array(bias), F)
        assert np.array_equal(F.numpy(), C.numpy())
        hip.dense(hip.array(a), hip.array(w), hip.array(bias), F, relu=True)
        R = hip.empty((m, n))
        hip.relu(C, R)
        assert np.array_equal(F.numpy(), R.numpy())
        hip.dense(hip.array(a), hip.array(w), None, F)
        hip.mult2D(hip.array(a), hip.array(w), R)
        assert np.array_equal(F.numpy(), R.numpy())
    x = rng.standard_normal((4, 1, 33, 31), dtype=np.float32) * 4
    B = hip.empty(x.shape)
    hip.sigmoid(hip.array(x), B)
    np.testing.assert_allclose(B.numpy(), oracle.sigmoid(x), rtol=1e-6, atol=1e-7)
    # line lengths on both sides of the 1024 entries the register path holds, axes with and without an inner stride
    for shape, axis in [((32, 1000), 1), ((3, 7, 5, 4), 1), ((6, 1), 1), ((5, 1024), 1), ((5, 1025), 1), ((3, 4099), 1), ((2, 1500, 3), 1),
                        ((2, 3, 70), 2)]:
        x = rng.standard_normal(shape, dtype=np.float32) * 3
        B = hip.empty(shape)
        hip.full_softmax(hip.array(x), B, axis)
        # the denominator is summed per lane and then across the wavefront, the oracle's sequentially: the two
        # orders drift apart with the length of the line (2e-6 up to 1024 entries, 5e-6 at 4099)
        np.testing.assert_allclose(B.numpy(), oracle.softmax(x, axis), rtol=2e-6 if shape[axis] <= 1024 else 5e-6, atol=1e-8)


def test_conv2d_cached_filters_follow_every_write(hip, oracle):
    """A registered filter tensor gives the results of an unregistered one, bit for bit, before and
    after its contents are replaced through the library (copy, fill, add, inc), and a freed
    tensor's entry does not outlive it."""
    rng = np.random.default_rng(415)
    N, C, H, W, Kf = 3, 24, 19, 17, 40
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    X = hip.array(x)

    def conv(Kd):
        O = hip.empty((N, Kf, H, W))
        hip.conv2D(X, Kd, None, O, 1, 1, 1, 1)
        return O.numpy()

    w1 = rng.standard_normal((Kf, C, 3, 3), dtype=np.float32)
    w2 = rng.standard_normal((Kf, C, 3, 3), dtype=np.float32)
    plain1, plain2 = conv(hip.array(w1)), conv(hip.array(w2))
    assert not np.array_equal(plain1, plain2)
    K = hip.array(w1)
    hip.cache_conv_filters(K)
    assert np.array_equal(conv(K), plain1)
    assert np.array_equal(conv(K), plain1)
    K.copy_from(w2)                                   # host -> device copy into the registered tensor
    assert np.array_equal(conv(K), plain2)
    hip.fill_(K, 0.0)
    assert not conv(K).any()
    hip.inc(hip.array(w1), K)                         # K += w1
    assert np.array_equal(conv(K), plain1)
    W2 = hip.array(w2)
    hip.add(1.0, W2, 0.0, W2, K)                      # K = w2 (+ 0*w2)
    assert np.array_equal(conv(K), plain2)
    with pytest.raises(Exception):
        hip._check(hip.lib.eddlhip_conv2d_cache_filters(hip.dev, K.ptr, Kf + 1, C, 3, 3))
    hip.uncache_conv_filters(K)
    assert np.array_equal(conv(K), plain2)
    # a registered tensor that is freed: the next tensor at that address starts unregistered
    hip.cache_conv_filters(K)
    del K
    for _ in range(4):
        K2 = hip.array(w1)
        assert np.array_equal(conv(K2), plain1)
        del K2
    hip.uncache_conv_filters(None)


def test_conv2d_random_shapes_against_oracle(hip, oracle):
    """120 seeded random problems: filter sides 1..7 (square and rectangular), strides 1..3, "same" /
    "valid" / custom symmetric pads, channel and filter counts that are not multiples of anything,
    batch 1..9, planes down to one pixel; whatever plan the planner picks."""
    rng = np.random.default_rng(417)
    done = 0
    while done < 120:
        R, S = (int(rng.integers(1, 8)),) * 2 if rng.random() < 0.7 else (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
        sr, sc = (int(rng.integers(1, 4)),) * 2 if rng.random() < 0.8 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        H, W = int(rng.integers(R, 40)), int(rng.integers(S, 40))
        N, C, Kf = int(rng.integers(1, 10)), int(rng.integers(1, 70)), int(rng.integers(1, 150))
        mode = rng.choice(["same", "valid", "custom"])
        pads = None
        if mode == "custom":
            pt, pl = int(rng.integers(0, R)), int(rng.integers(0, S))
            pads = [pt, pt, pl, pl]
        try:
            from eddl_amd.descriptors import ConvolDescriptor
            cd = ConvolDescriptor(Kf, [R, S], [sr, sc], str(mode), pads or [], use_bias=True).build([N, C, H, W])
        except RuntimeError:
            continue  # geometry the reference refuses (e.g. an empty output)
        if min(cd.out_shape) < 1:
            continue
        x = rng.standard_normal((N, C, H, W), dtype=np.float32)
        w = (rng.standard_normal((Kf, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
        b = rng.standard_normal(Kf, dtype=np.float32)
        ref, out = run_conv(hip, oracle, x, w, b, (sr, sc), str(mode), pads, relu=bool(done % 2))
        assert_conv_close(ref, out, "%s %s pads %s stride %s %s" % ((N, C, H, W, Kf, R, S), mode, pads, (sr, sc), hip.last_conv_kernel()))
        done += 1


def test_conv2d_input_beyond_2gib_runs_in_batch_chunks(hip, oracle):
    """An input of 2.7 GB is more than one buffer descriptor addresses: the launch is cut into batch
    chunks.  Sampled outputs from every chunk (first and last image included) against the oracle's
    direct form; the residual and the output pointers must advance with the chunks as well."""
    rng = np.random.default_rng(418)
    N, C, H, W, Kf = 42, 64, 512, 512, 4
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    b = rng.standard_normal(Kf, dtype=np.float32)
    res = rng.standard_normal((N, Kf, H, W), dtype=np.float32)
    O = hip.empty((N, Kf, H, W))
    hip.conv2D(hip.array(x), hip.array(w), hip.array(b), O, 1, 1, 1, 1, residual=hip.array(res))
    got = O.numpy()
    idx = np.stack([rng.integers(0, N, 4000), rng.integers(0, Kf, 4000), rng.integers(0, H, 4000), rng.integers(0, W, 4000)], 1)
    idx = np.concatenate([idx, [[0, 0, 0, 0], [N - 1, Kf - 1, H - 1, W - 1], [31, 1, 511, 511], [32, 2, 0, 0]]]).astype(np.int32)
    ref = oracle.conv2d_at(x, w, b, (1, 1), 1, 1, idx) + res[idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3]]
    pts = got[idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3]]
    tol = 1e-5 * float(np.abs(got).max()) + 1e-4 * np.abs(ref)
    assert np.all(np.abs(ref - pts) <= tol), np.abs(ref - pts).max()


def test_device_probes_report_plausible_rates(hip):
    from eddl_amd import EddlHipError
    rd, wr, cp = hip.probe_hbm(1 << 28)
    for v in (rd, wr, cp):
        assert 500.0 < v < 16000.0, (rd, wr, cp)   # GB/s: far above PCIe, below twice the published HBM peak
    with pytest.raises(EddlHipError, match="buffer size"):
        hip.probe_hbm(1000)
    mean, best, worst = hip.probe_mfma_f32(vary_operands=True, launches=3)
    assert 50.0 < worst <= mean <= best < 200.0


def test_conv2d_trace_records_one_timeline_per_workgroup(hip):
    """The measurement hook writes, per workgroup, four time stamps in order and where it ran; the output is unchanged."""
    rng = np.random.default_rng(5)
    x = hip.array(rng.standard_normal((8, 64, 28, 28), dtype=np.float32))
    w = hip.array((rng.standard_normal((64, 64, 3, 3)) * 0.05).astype(np.float32))
    O = hip.empty((8, 64, 28, 28))
    hip.conv2D(x, w, None, O, 1, 1, 1, 1, relu=True)
    plain = O.numpy()
    buf = hip.conv_trace(4096)
    try:
        hip.conv2D(x, w, None, O, 1, 1, 1, 1, relu=True)
        hip.synchronize()
    finally:
        hip.conv_trace(0)
    assert np.array_equal(O.numpy(), plain)
    rec = buf.numpy().view(np.uint64).reshape(-1, 8)
    rec = rec[rec[:, 0] != 0].astype(np.int64)
    assert len(rec) >= 8 * 28 * 28 // 128        # at least one workgroup per 64 x 128 tile of the largest tile shape
    t = rec[:, 0:4]
    assert np.all(np.diff(t, axis=1) >= 0)       # entry <= first operands in LDS <= end of the K loop <= stores drained
    assert np.all(t[:, 3] - t[:, 0] < 100_000_000)   # under a second of the 100 MHz clock
    assert np.all(rec[:, 6] > rec[:, 5])         # the shader clock advanced
    xcd = (rec[:, 4] >> 32) & 0xf
    assert len(np.unique(xcd)) == 8              # workgroups were dealt over all eight XCDs
    hip.conv2D(x, w, None, O, 1, 1, 1, 1, relu=True)   # switched off again: nothing is written
    hip.fill_(buf, 0.0)
    hip.conv2D(x, w, None, O, 1, 1, 1, 1, relu=True)
    hip.synchronize()
    assert not buf.numpy().any()


def test_conv2d_autotune_searches_once_per_geometry_and_stays_within_tolerance(hip, oracle):
    """With the plan search on, the first call of a geometry measures the launch plans and later calls reuse the choice;
    the result stays within the convolution's tolerance of the oracle and is the same from call to call, fused or not."""
    rng = np.random.default_rng(11)
    N, C, H, W, Kf = 8, 64, 28, 28, 64
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Kf, C, 3, 3)) * 0.05).astype(np.float32)
    g, b = rng.uniform(0.8, 1.2, Kf).astype(np.float32), (rng.standard_normal(Kf) * 0.1).astype(np.float32)
    mean, var = (rng.standard_normal(Kf) * 0.1).astype(np.float32), rng.uniform(0.5, 1.5, Kf).astype(np.float32)
    dx, dw = hip.array(x), hip.array(w)
    bn = (hip.array(g), hip.array(b), hip.array(mean), hip.array(var), 1e-5)
    O = hip.empty((N, Kf, H, W))
    hip.conv_autotune(-1)
    try:
        hip.conv_autotune(True)
        before = hip.conv_tuned_plans()
        hip.conv2D(dx, dw, None, O, 1, 1, 1, 1)
        after = hip.conv_tuned_plans()
        assert after in (before + 1, before + 2)             # the geometry itself, and the product launch of its Winograd form
        first = O.numpy()
        hip.conv2D(dx, dw, None, O, 1, 1, 1, 1)
        assert hip.conv_tuned_plans() == after               # same geometry: no second search
        assert np.array_equal(O.numpy(), first)
        ref = oracle.conv2d(x, w, None, (1, 1), 1, 1, H, W, algo="im2col")
        assert np.all(np.abs(first - ref) <= 1e-5 * float(np.abs(ref).max()) + 1e-4 * np.abs(ref))
        # the epilogue is not part of the geometry: conv + stand-alone batch norm == the fused call, bit for bit
        Y, opa, sd = hip.empty((N, Kf, H, W)), hip.empty((N, Kf, H, W)), hip.empty((Kf,))
        hip.batchnorm_inference(O, Y, opa, bn[2], bn[3], bn[0], bn[1], sd, 1e-5)
        F = hip.empty((N, Kf, H, W))
        hip.conv2D(dx, dw, None, F, 1, 1, 1, 1, bn=bn)
        assert hip.conv_tuned_plans() == after
        assert np.array_equal(F.numpy(), Y.numpy())
    finally:
        hip.conv_autotune(-1)
    assert hip.conv_tuned_plans() == 0
    hip.conv2D(dx, dw, None, O, 1, 1, 1, 1)
    assert hip.conv_tuned_plans() == 0                        # switched off: no search
