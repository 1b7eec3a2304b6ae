"""The CPU oracle against the vectors the reference's own unit tests hold, and against
what the mathematics fixes (library cross-checks, closed forms, invariants)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import eddl_allclose, tensor_of


def _conv_inputs(case):
    x = tensor_of(case["image"])
    C = x.shape[1]
    kshape = (case["filters"], C, case["kernel"][0], case["kernel"][1])
    w = np.ones(kshape, np.float32) if case["filters_data"] == "ones" else tensor_of(case["filters_data"])
    b = np.zeros(case["filters"], np.float32) if case["bias_data"] == "zeros" else tensor_of(case["bias_data"])
    return x, w, (b if case["use_bias"] else None)


def test_output_size_table(oracle, golden):
    t = golden["output_sizes"]
    i = 0
    for p in t["padding"]:
        for isz in t["input_sizes"]:
            for s in t["strides"]:
                for k in t["kernels"]:
                    assert oracle.out_size(p, isz, k, s) == t["output_sizes"][i], (p, isz, s, k)
                    i += 1
    assert i == 72


@pytest.mark.parametrize("algo", ["direct", "im2col"])
def test_conv2d_reference_vectors(oracle, golden, algo):
    for case in golden["conv2d"]:
        x, w, b = _conv_inputs(case)
        H, W = x.shape[2:]
        P, Q, pads = oracle.conv_geometry(H, W, *case["kernel"], *case["strides"], case["padding"])
        exp = tensor_of(case["forward"])
        assert (1, case["filters"], P, Q) == exp.shape, case["name"]
        out = oracle.conv2d(x, w, b, case["strides"], pads[0], pads[2], P, Q, algo=algo)
        assert eddl_allclose(exp, out, case["atol"], case["rtol"]), case["name"]
        # integer data: any summation order is exact
        assert np.array_equal(exp, out), case["name"]


def test_conv2d_backward_maps_pin_the_taps(oracle, golden):
    """The reference's backward-of-ones vectors equal sum over outputs of the filter taps that
    touched each input pixel; rebuilding them from the forward geometry pins pad/stride
    placement (which taps exist) independently of the forward values."""
    for case in golden["conv2d"]:
        x, w, _ = _conv_inputs(case)
        _, C, H, W = x.shape
        R, S = case["kernel"]
        sr, sc = case["strides"]
        P, Q, pads = oracle.conv_geometry(H, W, R, S, sr, sc, case["padding"])
        back = np.zeros_like(x)
        for k in range(case["filters"]):
            for p in range(P):
                for q in range(Q):
                    for c in range(C):
                        for r in range(R):
                            for s in range(S):
                                y, xx = p * sr + r - pads[0], q * sc + s - pads[2]
                                if 0 <= y < H and 0 <= xx < W:
                                    back[0, c, y, xx] += w[k, c, r, s]
        assert np.array_equal(back, tensor_of(case["backward_of_ones"])), case["name"]


@pytest.mark.parametrize("shape", [
    # N, C, H, W, Kf, R, S, sr, sc, padding
    (2, 3, 9, 11, 4, 3, 3, 1, 1, "same"),
    (2, 5, 10, 7, 3, 3, 3, 2, 2, "same"),      # asymmetric same pads (0,1)
    (1, 4, 12, 12, 6, 1, 1, 2, 2, "valid"),
    (2, 2, 13, 9, 3, 7, 7, 2, 2, "same"),      # asymmetric same pads (2,3)
    (1, 3, 8, 8, 2, 2, 2, 1, 1, "valid"),
    (3, 6, 6, 5, 5, 3, 2, 1, 2, "same"),
])
def test_conv2d_against_torch(oracle, shape):
    N, C, H, W, Kf, R, S, sr, sc, padding = shape
    rng = np.random.default_rng(7)
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = rng.standard_normal((Kf, C, R, S), dtype=np.float32)
    b = rng.standard_normal(Kf, dtype=np.float32)
    P, Q, (pt, pb, pl, pr) = oracle.conv_geometry(H, W, R, S, sr, sc, padding)
    xt = F.pad(torch.from_numpy(x).double(), (pl, pr, pt, pb))
    ref = F.conv2d(xt, torch.from_numpy(w).double(), torch.from_numpy(b).double(), stride=(sr, sc)).numpy()
    assert ref.shape == (N, Kf, P, Q)
    for algo in ("direct", "im2col"):
        out = oracle.conv2d(x, w, b, (sr, sc), pt, pl, P, Q, algo=algo)
        np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-4)
    idx = np.array([[n, k, p, q] for n in range(N) for k in (0, Kf - 1) for p in (0, P - 1) for q in (0, Q // 2, Q - 1)], np.int32)
    at = oracle.conv2d_at(x, w, b, (sr, sc), pt, pl, idx)
    full = oracle.conv2d(x, w, b, (sr, sc), pt, pl, P, Q)
    assert np.array_equal(at, full[idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3]])


def _pool_setup(oracle, case):
    x = tensor_of(case["image"])
    H, W = x.shape[2:]
    r, c, pads, lp, lq = oracle.pool_geometry(H, W, *case["kernel"], *case["strides"], case["padding"])
    assert (r, c) == (lp, lq), case["name"]
    return x, pads


def test_maxpool_reference_vectors(oracle, golden):
    for case in golden["maxpool2d"]:
        x, pads = _pool_setup(oracle, case)
        O, ix, iy = oracle.maxpool2d(x, case["kernel"], case["strides"], pads)
        exp = tensor_of(case["forward"])
        assert O.shape == exp.shape, case["name"]
        assert np.array_equal(O, exp), case["name"]
        # the reference's backward-of-ones map is the histogram of (indY, indX): this pins
        # the argmax convention (absolute coordinates, first maximum wins in (ky,kx) order)
        hist = np.zeros_like(x)
        for yy, xx in zip(iy.ravel(), ix.ravel()):
            hist[0, 0, int(yy), int(xx)] += 1
        assert np.array_equal(hist, tensor_of(case["backward_of_ones"])), case["name"]


def test_maxpool_against_torch(oracle):
    rng = np.random.default_rng(11)
    for (H, W, k, s, p) in [(12, 10, 2, 2, 0), (9, 9, 3, 2, 1), (8, 14, 3, 1, 1), (7, 7, 7, 1, 0)]:
        x = rng.integers(-4, 5, size=(2, 3, H, W)).astype(np.float32)  # many exact ties
        O, ix, iy = oracle.maxpool2d(x, (k, k), (s, s), (p, p, p, p))
        to, ti = F.max_pool2d(torch.from_numpy(x), k, s, p, return_indices=True)
        assert np.array_equal(O, to.numpy())
        # torch breaks ties towards the first maximum in row-major window order too
        assert np.array_equal(iy * W + ix, ti.numpy().astype(np.float32))


def test_maxpool_untouched_indices_and_floor(oracle):
    x = np.full((1, 1, 4, 4), -np.inf, np.float32)
    x[0, 0, 2:, 2:] = np.nan
    O, ix, iy = oracle.maxpool2d(x, (2, 2), (2, 2), (0, 0, 0, 0), fill=-7.0)
    assert np.all(O == np.float32(-3.40282e38))   # running maximum never replaced
    assert np.all(ix == -7.0) and np.all(iy == -7.0)  # index slots left as they were


def test_avgpool_reference_vectors(oracle, golden):
    for case in golden["avgpool2d"]:
        x, pads = _pool_setup(oracle, case)
        O = oracle.avgpool2d(x, case["kernel"], case["strides"], pads)
        exp = tensor_of(case["forward"])
        assert O.shape == exp.shape, case["name"]
        assert eddl_allclose(exp, O, case["atol"], case["rtol"]), case["name"]


def test_avgpool_against_torch(oracle):
    rng = np.random.default_rng(12)
    for (H, W, k, s, p) in [(12, 10, 2, 2, 0), (9, 9, 3, 2, 1), (8, 14, 3, 1, 1), (7, 7, 7, 1, 0)]:
        x = rng.standard_normal((2, 3, H, W), dtype=np.float32)
        O = oracle.avgpool2d(x, (k, k), (s, s), (p, p, p, p))
        ref = F.avg_pool2d(torch.from_numpy(x).double(), k, s, p, count_include_pad=True).numpy()
        np.testing.assert_allclose(O, ref, rtol=1e-5, atol=1e-6)


def test_pool_custom_pad_column_count_uses_row_pads(oracle):
    # descriptor_pool2D.cpp:69-70 hands the 4-vector to compute_output, which reads [0],[1]
    r, c, pads, lp, lq = oracle.pool_geometry(10, 10, 3, 3, 2, 2, "custom", (1, 1, 0, 0))
    assert (r, c) == (5, 5) and (lp, lq) == (5, 4)


def test_pad_reference_vector(oracle, golden):
    case = golden["pad"]
    out = oracle.pad(tensor_of(case["input"]), case["pads"])
    assert eddl_allclose(tensor_of(case["expected"]), out, case["atol"])


def test_pad_order_top_right_bottom_left(oracle):
    x = np.arange(6, dtype=np.float32).reshape(1, 1, 2, 3)
    out = oracle.pad(x, (1, 2, 3, 4), cval=9.0)
    assert out.shape == (1, 1, 2 + 1 + 3, 3 + 4 + 2)
    ref = F.pad(torch.from_numpy(x), (4, 2, 1, 3), value=9.0).numpy()
    assert np.array_equal(out, ref)


def test_softmax_reference_vector(oracle, golden):
    case = golden["softmax"]
    out = oracle.softmax(tensor_of(case["input"]), case["axis"])
    assert eddl_allclose(tensor_of(case["expected"]), out, case["atol"])


def test_softmax_against_torch_and_eps_seed(oracle):
    rng = np.random.default_rng(13)
    x = rng.standard_normal((4, 10), dtype=np.float32) * 3
    out = oracle.softmax(x, 1)
    ref = torch.softmax(torch.from_numpy(x).double(), 1).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-7)
    # single-element axis: exp(0)=1 divided by (1.19209e-07 + 1)
    one = oracle.softmax(np.zeros((3, 1), np.float32), 1)
    assert np.all(one == np.float32(1.0) / (np.float32(1.19209e-07) + np.float32(1.0)))
    x4 = rng.standard_normal((2, 5, 3, 4), dtype=np.float32)
    np.testing.assert_allclose(oracle.softmax(x4, 1), torch.softmax(torch.from_numpy(x4).double(), 1).numpy(), rtol=1e-5, atol=1e-7)


def test_batchnorm_inference_closed_form(oracle):
    rng = np.random.default_rng(14)
    x = rng.standard_normal((3, 5, 4, 6), dtype=np.float32)
    mean = (rng.standard_normal(5) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, 5).astype(np.float32)
    g = rng.uniform(0.8, 1.2, 5).astype(np.float32)
    b = (rng.standard_normal(5) * 0.1).astype(np.float32)
    eps = 1e-5
    y, opa, sd = oracle.batchnorm_inference(x, mean, var, g, b, eps)
    ref = F.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(mean).double(), torch.from_numpy(var).double(),
                       torch.from_numpy(g).double(), torch.from_numpy(b).double(), False, 0.0, eps).numpy()
    np.testing.assert_allclose(y, ref, rtol=2e-6, atol=2e-6)
    assert np.array_equal(sd, np.sqrt(var + np.float32(eps)))
    # the written rounding sequence, step by step in float32
    m4, s4, g4, b4 = (v.reshape(1, 5, 1, 1) for v in (mean, sd, g, b))
    o = (x - m4) / s4
    assert np.array_equal(opa, o)
    assert np.array_equal(y, o * g4 + b4)
    # identity invariant: mean 0, var = 1-eps, gamma 1, beta 0  =>  y == x
    eps2 = np.float32(0.25)
    y2, _, _ = oracle.batchnorm_inference(x, np.zeros(5, np.float32), np.full(5, 0.75, np.float32),
                                          np.ones(5, np.float32), np.zeros(5, np.float32), float(eps2))
    assert np.array_equal(y2, x)
    # no affine
    y3, opa3, _ = oracle.batchnorm_inference(x, mean, var, None, None, eps)
    assert opa3 is None and np.array_equal(y3, o)


def test_relu_edge_cases(oracle):
    x = np.array([-1.0, -0.0, 0.0, 2.5, np.nan, np.inf, -np.inf, 1e-45], np.float32)
    y = oracle.relu(x)
    assert np.array_equal(y, np.array([0, 0, 0, 2.5, 0, np.inf, 0, 1e-45], np.float32))
    assert not np.signbit(y[1]) and not np.signbit(y[4])


def test_sigmoid_add_concat_upsample_dense(oracle):
    rng = np.random.default_rng(15)
    x = rng.standard_normal((2, 3, 4, 5), dtype=np.float32)
    np.testing.assert_allclose(oracle.sigmoid(x), torch.sigmoid(torch.from_numpy(x).double()).numpy(), rtol=1e-6, atol=1e-7)
    y = rng.standard_normal((2, 3, 4, 5), dtype=np.float32)
    assert np.array_equal(oracle.add(x, y), x + y)
    assert np.array_equal(oracle.add(x, y, 2.0, -0.5), np.float32(2.0) * x + np.float32(-0.5) * y)
    assert np.array_equal(oracle.add(x, y, c=x), x + (x + y))
    z = rng.standard_normal((2, 7, 4, 5), dtype=np.float32)
    for axis, parts in [(1, [x, z, y]), (0, [x, y]), (3, [x, y])]:
        assert np.array_equal(oracle.concat(parts, axis), np.concatenate(parts, axis))
    for s in (2, 3):
        up = oracle.scale_nearest(x, (4 * s, 5 * s))
        ref = F.interpolate(torch.from_numpy(x), scale_factor=s, mode="nearest").numpy()
        assert np.array_equal(up, ref)
        assert np.array_equal(up, x.repeat(s, 2).repeat(s, 3))
    a = rng.standard_normal((5, 37), dtype=np.float32)
    w = rng.standard_normal((37, 300), dtype=np.float32)
    bias = rng.standard_normal(300, dtype=np.float32)
    np.testing.assert_allclose(oracle.dense(a, w, bias), a.astype(np.float64) @ w.astype(np.float64) + bias, rtol=1e-4, atol=1e-4)
