"""ONNX import / export of the forward path, on the CPU.

What pins the importer: three files written by PyTorch's exporter (tests/golden/onnx/*.onnx, made by
tests/golden/make_onnx_fixtures.py) with PyTorch's own outputs for a seeded input.  The imported
graph is run on the CPU oracle and has to reproduce those outputs, which also cross-checks the
oracle's batch norm, pools, upsampling, pad, concat, dense, softmax and sigmoid against a second,
unrelated implementation.  The repairs the reference's importer makes (asymmetric paddings, constants
added onto a layer) are exercised with small files written by this package's own encoder.
"""
import os

import numpy as np
import pytest

from eddl_amd import models, onnx_io as O
from eddl_amd import net as N
from oracle import net_oracle

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = os.path.join(HERE, "golden", "onnx")

EXPECTED_KINDS = {
    "vgg_like": ["input", "conv2d", "relu", "maxpool2d", "conv2d", "relu", "batchnorm", "avgpool2d", "reshape", "dense", "relu", "dense",
                 "softmax"],
    "resnet_like": ["input", "conv2d", "relu", "maxpool2d", "conv2d", "relu", "conv2d", "add_n", "relu", "conv2d", "relu", "conv2d",
                    "conv2d", "add_n", "relu", "avgpool2d", "reshape", "dense"],
    "unet_like": ["input", "conv2d", "relu", "maxpool2d", "conv2d", "relu", "resize", "pad", "conv2d", "concat", "conv2d", "relu",
                  "conv2d", "sigmoid"],
}


def close(ref, out):
    ref = np.asarray(ref, np.float32)
    return bool(np.all(np.abs(ref - out) <= 1e-5 * np.abs(ref).max() + 1e-4 * np.abs(ref)))


# ---------------------------------------------------------------------------- wire format
def test_varints_and_packed_fields_round_trip():
    for v in (0, 1, 127, 128, 300, 2**31 - 1, 2**63 - 1, -1, -2**63):
        got, pos = O._varint(O._wvarint(v), 0)
        assert O._signed(got) == v and pos == len(O._wvarint(v))
    # 300 is the two bytes AC 02 in every protobuf text
    assert O._wvarint(300) == b"\xac\x02"
    # an attribute with negative and large ints, packed as this encoder writes them and unpacked as older writers do
    packed = O.AttributeProto(O._attr("pads", [0, -1, 2**40, 3]))
    assert packed.name == "pads" and packed.ints == [0, -1, 2**40, 3]
    unpacked = O._wbytes(1, "pads") + b"".join(O._wint(8, v) for v in [0, -1, 2**40, 3])
    assert O.AttributeProto(unpacked).ints == [0, -1, 2**40, 3]
    a = O.AttributeProto(O._attr("epsilon", 1e-5))
    assert a.f == np.float32(1e-5)
    assert O.AttributeProto(O._attr("mode", "nearest")).s == "nearest"


def test_tensor_encodings():
    w = np.arange(24, dtype=np.float32).reshape(2, 3, 4) - 7.5
    t = O.TensorProto(O._tensor("w", w))
    assert t.name == "w" and t.dims == [2, 3, 4] and t.data_type == O.FLOAT and np.array_equal(t.values, w.ravel())
    # raw_data, the form PyTorch writes
    raw = O._wbytes(1, O._wvarint(2) + O._wvarint(2)) + O._wint(2, O.FLOAT) + O._wbytes(9, np.float32([1, -2, 3.5, 4]).tobytes())
    assert np.array_equal(O.TensorProto(raw).values, np.float32([1, -2, 3.5, 4]))
    # int64 tensors (shapes, paddings) come out as floats, as in the reference's initializer maps
    i = O.TensorProto(O._tensor("shape", np.array([-1, 128], np.int64), O.INT64))
    assert i.data_type == O.INT64 and list(i.values) == [-1.0, 128.0]
    raw64 = O._wbytes(1, O._wvarint(3)) + O._wint(2, O.INT64) + O._wbytes(9, np.array([0, -3, 2**33], np.int64).tobytes())
    assert list(O.TensorProto(raw64).values) == [0.0, -3.0, float(2**33)]
    scalar = O.TensorProto(O._tensor("c", np.array(0.25, np.float32)))
    assert scalar.dims == [] and list(scalar.values) == [0.25]


def test_truncated_and_missing_files(tmp_path):
    data = open(os.path.join(FIX, "vgg_like.onnx"), "rb").read()
    with pytest.raises(RuntimeError, match="ONNX::ImportNet"):
        O.import_net_from_onnx_bytes(data[:len(data) // 2])
    with pytest.raises(RuntimeError, match="ONNX::ImportNet"):
        O.import_net_from_onnx_file(str(tmp_path / "absent.onnx"))


# ---------------------------------------------------------------------------- files written by PyTorch
@pytest.mark.parametrize("name", sorted(EXPECTED_KINDS))
def test_pytorch_files_import_and_reproduce_pytorch_outputs(oracle, name):
    net = O.import_net_from_onnx_file(os.path.join(FIX, name + ".onnx"))
    d = np.load(os.path.join(FIX, name + ".npz"))
    assert [l.kind for l in net.layers] == EXPECTED_KINDS[name]
    assert net.lin[0].out_shape == [1] + list(d["x"].shape[1:])  # batch 1 until a forward says otherwise
    y = net_oracle.forward(oracle, net, [d["x"]], conv_algo="direct")[0]
    assert y.shape == d["y"].shape
    assert close(d["y"], y), np.abs(y - d["y"]).max()


def test_details_of_the_imported_layers():
    net = O.import_net_from_onnx_file(os.path.join(FIX, "vgg_like.onnx"))
    by_kind = {}
    for l in net.layers:
        by_kind.setdefault(l.kind, []).append(l)
    c1, c2 = by_kind["conv2d"]
    assert c1.attrs["cd"].use_bias and not c2.attrs["cd"].use_bias
    assert c1.attrs["cd"].pads == [1, 1, 1, 1] and c1.params["K"].shape == (6, 3, 3, 3)
    bn = by_kind["batchnorm"][0]
    assert bn.attrs["affine"] and abs(bn.attrs["epsilon"] - 1e-5) < 1e-12 and abs(bn.attrs["momentum"] - 0.9) < 1e-6
    assert list(bn.params) == ["bn_g", "bn_b", "mean", "variance"] and bn.params["variance"].min() >= 0.5
    d1, d2 = by_kind["dense"]
    assert d1.params["W"].shape == (128, 12) and d2.params["W"].shape == (12, 5)  # transB = 1 in the file: [out, in] -> [in, out]
    assert by_kind["softmax"][0].attrs["axis"] == 1
    # the ResNet-like file: 3x3 stride-2 max-pool with paddings 1, GlobalAveragePool as an average pool over the plane
    net = O.import_net_from_onnx_file(os.path.join(FIX, "resnet_like.onnx"))
    mp = [l for l in net.layers if l.kind == "maxpool2d"][0].attrs["pd"]
    assert (mp.kr, mp.kc, mp.sr, mp.sc, mp.pad) == (3, 3, 2, 2, [1, 1, 1, 1])
    gap = [l for l in net.layers if l.kind == "avgpool2d"][0]
    assert gap.attrs["pd"].ksize == gap.parents[0].out_shape[2:] and gap.out_shape[2:] == [1, 1]
    # the U-Net-like file: Upsample by 2, Pad (bottom 1, right 1) as (top, right, bottom, left), concat over the channels
    net = O.import_net_from_onnx_file(os.path.join(FIX, "unet_like.onnx"))
    pad = [l for l in net.layers if l.kind == "pad"][0]
    assert pad.attrs["pads"] == [0, 1, 1, 0] and pad.attrs["constant"] == 0.0
    rs = [l for l in net.layers if l.kind == "resize"][0]
    assert rs.out_shape[2:] == [2 * d for d in rs.parents[0].out_shape[2:]]
    assert [l for l in net.layers if l.kind == "concat"][0].attrs["axis"] == 1


def test_input_shape_override():
    net = O.import_net_from_onnx_file(os.path.join(FIX, "unet_like.onnx"), input_shape=[1, 32, 48])
    assert net.lin[0].out_shape == [1, 1, 32, 48] and net.lout[0].out_shape == [1, 1, 32, 48]


# ---------------------------------------------------------------------------- export -> import
@pytest.mark.parametrize("which", ["block", "vgg16", "resnet50", "unet"])
def test_export_import_round_trip(which):
    if which == "block":
        m = models.conv_bn_relu_pool_block(batch=1, channels=5, size=12, filters=7)
    elif which == "vgg16":
        m = models.vgg16(batch=1, size=32, num_classes=10, widths=(4, 8, 8, 16, 16), dense=32)
    elif which == "resnet50":
        m = models.resnet50(batch=1, size=64, num_classes=10, base=4)
    else:
        m = models.unet(batch=1, size=32, widths=(4, 8), bottleneck=16)
    models.init_he_normal(m, 5)
    data = O.export_net_to_onnx_bytes(m)
    model = O.ModelProto(data)
    assert model.producer_name == "EDDL" and model.opset_import == [("", 11)] and model.graph.name == "Computational Graph"
    assert model.graph.input[0].dims[0] == "batch" and model.graph.input[0].dims[1:] == m.lin[0].out_shape[1:]
    back = O.import_net_from_onnx_bytes(data)
    # LSum comes back as LSum (Sum node), everything else as itself; names are the layers' names
    assert [(l.kind, l.name, l.out_shape) for l in back.layers] == [(l.kind, l.name, l.out_shape) for l in m.layers]
    for a, b in zip(m.layers, back.layers):
        assert list(a.params) == list(b.params)
        for key in a.params:
            used = key != "bias" or (a.attrs["cd"].use_bias if a.kind == "conv2d" else a.attrs.get("use_bias", True))
            if used:
                assert np.array_equal(a.params[key], b.params[key]), (a.name, key)
        if a.kind == "conv2d":
            ca, cb = a.attrs["cd"], b.attrs["cd"]
            assert (ca.pads, ca.sr, ca.sc, ca.use_bias) == (cb.pads, cb.sr, cb.sc, cb.use_bias)
        if a.kind == "batchnorm":
            assert abs(a.attrs["epsilon"] - b.attrs["epsilon"]) < 1e-12
        if a.kind == "pad":
            assert a.attrs["pads"] == b.attrs["pads"]
    # parameters are written as float_data, the form the reference's exporter uses (no raw_data field 9 in an initializer)
    for f, wt, v in O._fields(next(v for f, wt, v in O._fields(data) if f == 7)):
        if f == 5:
            assert 9 not in [f2 for f2, _, _ in O._fields(v)]


# ---------------------------------------------------------------------------- the importer's repairs
def tiny_model(nodes, inits, in_shape, out_name, out_shape):
    graph = b"".join(O._wbytes(1, n) for n in nodes) + b"".join(O._wbytes(5, t) for t in inits)
    graph += O._wbytes(11, O._value_info("x", [1] + in_shape)) + O._wbytes(12, O._value_info(out_name, [1] + out_shape))
    return O._wint(1, 6) + O._wbytes(7, graph) + O._wbytes(8, O._wint(2, 11))


def test_asymmetric_paddings_become_a_pad_layer(oracle):
    rng = np.random.default_rng(3)
    K = rng.standard_normal((4, 2, 2, 2)).astype(np.float32)
    conv = O._node("Conv", "c", ["x", "c_W"], ["c"], [("kernel_shape", [2, 2]), ("pads", [0, 0, 1, 1]), ("strides", [1, 1])])
    pool = O._node("MaxPool", "p", ["c"], ["p"], [("kernel_shape", [2, 2]), ("pads", [1, 0, 0, 1]), ("strides", [2, 2])])
    net = O.import_net_from_onnx_bytes(tiny_model([conv, pool], [O._tensor("c_W", K)], [2, 6, 6], "p", [4, 3, 3]))
    assert [(l.kind, l.name) for l in net.layers] == [("input", "x"), ("pad", "c__asymmetric_padding"), ("conv2d", "c"),
                                                      ("pad", "p__asymmetric_padding"), ("maxpool2d", "p")]
    pads = [l.attrs["pads"] for l in net.layers if l.kind == "pad"]
    assert pads == [[0, 1, 1, 0], [1, 1, 0, 0]]  # (top, right, bottom, left)
    assert net.layers[2].attrs["cd"].pads == [0, 0, 0, 0] and net.layers[2].out_shape == [1, 4, 6, 6]
    assert net.layers[1].children == [net.layers[2]] and net.layers[0].children == [net.layers[1]]  # the refused layers left no trace
    # the convolution with a zero border on the bottom and right equals the padded "valid" convolution
    x = rng.standard_normal((1, 2, 6, 6)).astype(np.float32)
    y = net_oracle.forward(oracle, net, [x], conv_algo="direct", keep=True)[1]["c"]
    want = oracle.conv2d(np.pad(x, ((0, 0), (0, 0), (0, 1), (0, 1))), K, None, (1, 1), 0, 0, 6, 6, algo="direct")
    assert np.array_equal(y, want)


def test_constants_added_onto_layers_become_biases():
    rng = np.random.default_rng(4)
    K, b0, b1 = rng.standard_normal((3, 2, 1, 1)).astype(np.float32), np.float32([1, 2, 3]), np.float32([0.5, 0.25, 0.125])
    W, wb = rng.standard_normal((27, 4)).astype(np.float32), np.float32([1, -1, 2, -2])
    nodes = [O._node("Conv", "c", ["x", "K"], ["c"], [("kernel_shape", [1, 1])]),
             O._node("Add", "a0", ["c", "b0"], ["a0"]),      # no bias yet: becomes the bias
             O._node("Add", "a1", ["b1", "a0"], ["a1"]),     # constant on the left, bias present: added to it
             O._node("Flatten", "f", ["a1"], ["f"]),
             O._node("MatMul", "mm", ["f", "W"], ["mm"]),
             O._node("Add", "a2", ["mm", "wb"], ["a2"])]
    inits = [O._tensor("K", K), O._tensor("b0", b0), O._tensor("b1", b1), O._tensor("W", W), O._tensor("wb", wb)]
    net = O.import_net_from_onnx_bytes(tiny_model(nodes, inits, [2, 3, 3], "a2", [4]))
    assert [l.kind for l in net.layers] == ["input", "conv2d", "reshape", "dense"]
    conv, dense = net.layers[1], net.layers[3]
    assert conv.attrs["cd"].use_bias and np.array_equal(conv.params["bias"], b0 + b1)
    assert dense.attrs["use_bias"] and np.array_equal(dense.params["bias"], wb) and np.array_equal(dense.params["W"], W)
    assert net.lout == [dense]


def test_nodes_outside_the_path_are_refused():
    node = O._node("LSTM", "r", ["x"], ["r"])
    with pytest.raises(RuntimeError, match="ONNX::ImportNet"):
        O.import_net_from_onnx_bytes(tiny_model([node], [], [4, 4], "r", [4]))
    up = O._node("Resize", "u", ["x", "", "s"], ["u"], [("mode", "linear")])
    with pytest.raises(RuntimeError, match="ONNX::ImportNet"):
        O.import_net_from_onnx_bytes(tiny_model([up], [O._tensor("s", np.float32([1, 1, 2, 2]))], [1, 4, 4], "u", [1, 8, 8]))
    cat = O._node("Concat", "k", ["x", "x"], ["k"], [("axis", 0)])
    with pytest.raises(RuntimeError, match="ONNX::ImportNet"):
        O.import_net_from_onnx_bytes(tiny_model([cat], [], [1, 4, 4], "k", [1, 4, 4]))


def test_pools_refuse_asymmetric_paddings_like_the_reference():
    x = N.Input([3, 5, 5])
    with pytest.raises(N.AsymmetricPaddingException) as e:
        N.MaxPool2D(x, [2, 2], [2, 2], "same")
    assert e.value.pads == [0, 1, 0, 1]
    with pytest.raises(N.AsymmetricPaddingException):
        N.AveragePool2D(x, [2, 2], [2, 2], [0, 1, 0, 1])


# ---------------------------------------------------------------------------- the C++ importer / exporter (host only)
NET_DRIVER = os.path.join(os.path.dirname(HERE), "eddl_amd", "host", "net_driver")


def cpp_onnxinfo(path, back=None):
    import subprocess
    if not os.path.exists(NET_DRIVER):
        subprocess.run(["make", "-C", os.path.dirname(NET_DRIVER), "all"], check=True, stdout=subprocess.DEVNULL)
    res = subprocess.run([NET_DRIVER, "onnxinfo", str(path)] + ([str(back)] if back else []), stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=120)
    return res


def layer_lines(net):
    """What `net_driver onnxinfo` prints for a net, computed from the Python graph."""
    out = []
    for l in net.layers:
        fields = ["layer", l.kind, l.name] + [str(d) for d in l.out_shape]
        line = " ".join(fields)
        for key, v in l.params.items():
            if key == "bias" and l.kind == "dense" and not l.attrs["use_bias"]:
                continue  # the C++ LDense owns no bias tensor then
            line += " | %d %.9g" % (v.size, float(np.sum(v.astype(np.float64))))
        out.append(line)
    return out


@pytest.mark.parametrize("name", sorted(EXPECTED_KINDS))
def test_cpp_importer_builds_the_same_graph_as_the_python_importer(name, tmp_path):
    path = os.path.join(FIX, name + ".onnx")
    res = cpp_onnxinfo(path, tmp_path / "back.onnx")
    assert res.returncode == 0, res.stderr[-2000:]
    want = layer_lines(O.import_net_from_onnx_file(path))
    got = [l for l in res.stdout.splitlines() if l.startswith("layer ")]
    assert len(got) == len(want)
    for g, w in zip(got, want):
        gk, wk = g.split(" | "), w.split(" | ")
        assert gk[0] == wk[0] and len(gk) == len(wk), (g, w)
        for a, b in zip(gk[1:], wk[1:]):  # parameter size exact, sum of values to float printing
            assert a.split()[0] == b.split()[0] and abs(float(a.split()[1]) - float(b.split()[1])) <= 1e-6 * max(1.0, abs(float(b.split()[1]))), (g, w)
    # what the C++ exporter wrote comes back through the Python importer with the same layers and parameters
    net, back = O.import_net_from_onnx_file(path), O.import_net_from_onnx_file(str(tmp_path / "back.onnx"))
    assert [(l.kind, l.name, l.out_shape) for l in back.layers] == [(l.kind, l.name, l.out_shape) for l in net.layers]
    for a, b in zip(net.layers, back.layers):
        for key in a.params:
            if key == "bias" and not (a.attrs["cd"].use_bias if a.kind == "conv2d" else a.attrs.get("use_bias", True)):
                continue
            assert np.array_equal(a.params[key], b.params[key]), (a.name, key)


def test_cpp_importer_repairs_and_errors(tmp_path):
    rng = np.random.default_rng(6)
    K = rng.standard_normal((4, 2, 2, 2)).astype(np.float32)
    conv = O._node("Conv", "c", ["x", "c_W"], ["c"], [("kernel_shape", [2, 2]), ("pads", [0, 0, 1, 1]), ("strides", [1, 1])])
    add = O._node("Add", "a", ["c", "b"], ["a"])
    pool = O._node("AveragePool", "p", ["a"], ["p"], [("kernel_shape", [2, 2]), ("pads", [1, 0, 0, 1]), ("strides", [2, 2])])
    data = tiny_model([conv, add, pool], [O._tensor("c_W", K), O._tensor("b", np.float32([1, 2, 3, 4]))], [2, 6, 6], "p", [4, 3, 3])
    (tmp_path / "m.onnx").write_bytes(data)
    res = cpp_onnxinfo(tmp_path / "m.onnx")
    assert res.returncode == 0, res.stderr[-2000:]
    want = layer_lines(O.import_net_from_onnx_bytes(data))
    assert [l for l in res.stdout.splitlines() if l.startswith("layer ")] == want
    assert [w.split()[1:3] for w in want] == [["input", "x"], ["pad", "c__asymmetric_padding"], ["conv2d", "c"],
                                             ["pad", "p__asymmetric_padding"], ["avgpool2d", "p"]]
    assert want[2].endswith("| 4 10")  # the added constant became the convolution's bias
    # refused nodes and broken files raise the reference's error, not a crash
    (tmp_path / "bad.onnx").write_bytes(tiny_model([O._node("LSTM", "r", ["x"], ["r"])], [], [4, 4], "r", [4]))
    res = cpp_onnxinfo(tmp_path / "bad.onnx")
    assert res.returncode == 1 and "ONNX::ImportNet" in res.stderr
    (tmp_path / "cut.onnx").write_bytes(open(os.path.join(FIX, "vgg_like.onnx"), "rb").read()[:3000])
    res = cpp_onnxinfo(tmp_path / "cut.onnx")
    assert res.returncode == 1 and "ONNX::ImportNet" in res.stderr
    res = cpp_onnxinfo(tmp_path / "absent.onnx")
    assert res.returncode == 1 and "ONNX::ImportNet" in res.stderr


def random_net(rng):
    """A small random graph over the layer set of the path (valid shapes by construction)."""
    c, size = int(rng.integers(1, 5)), int(rng.integers(9, 17))
    x = N.Input([c, size, size])
    l, skips = x, []
    for _ in range(int(rng.integers(3, 9))):
        choice = rng.integers(0, 10)
        h = l.out_shape[2]
        if choice == 0 and h >= 6:
            k = int(rng.integers(1, 4))
            l = N.Conv2D(l, int(rng.integers(1, 7)), [k, k], [1, 1], "custom", bool(rng.integers(0, 2)), pads=[k // 2] * 4)
        elif choice == 1 and h >= 6:
            l = N.Conv2D(l, int(rng.integers(1, 7)), [3, 3], [2, 2], "custom", True, pads=[1, 1, 1, 1])
        elif choice == 2:
            l = N.BatchNormalization(l, True, 0.9, float(rng.choice([1e-5, 1e-3])))
        elif choice == 3:
            l = N.ReLu(l)
        elif choice == 4 and h >= 4:
            l = (N.MaxPool2D if rng.integers(0, 2) else N.AveragePool2D)(l, [2, 2], [2, 2], [0, 0, 0, 0])
        elif choice == 7:
            l = N.BatchNormalization(N.ReLu(l), True, 0.9, 1e-5)  # two shape-keeping layers: partners for a later add / concat
        elif choice == 5 and h <= 12:
            l = N.UpSampling2D(l, [2, 2])
        elif choice == 6:
            l = N.Pad(l, [int(v) for v in rng.integers(0, 3, 4)], 0.0)
        else:
            same = [s for s in skips if s.out_shape == l.out_shape and s is not l]
            if same:
                l = N.Add(l, same[0]) if rng.integers(0, 2) else N.Concat([l, same[0]])
            else:
                l = N.Sigmoid(l)
        skips.append(l)
    l = N.Dense(N.Flatten(l), int(rng.integers(2, 6)), bool(rng.integers(0, 2)))
    net = N.Net([x], [N.Softmax(l)])
    for layer in net.layers:
        for key, v in layer.params.items():
            w = rng.standard_normal(v.shape).astype(np.float32)
            layer.params[key] = np.abs(w) + 0.5 if key == "variance" else w * np.float32(0.5)
    return net


@pytest.mark.parametrize("seed", range(30))
def test_random_graphs_through_both_codecs(seed, tmp_path):
    """Python export -> C++ import -> C++ export -> Python import: the same layers, shapes and parameters all the way."""
    net = random_net(np.random.default_rng(100 + seed))
    data = O.export_net_to_onnx_bytes(net)
    (tmp_path / "a.onnx").write_bytes(data)
    res = cpp_onnxinfo(tmp_path / "a.onnx", tmp_path / "b.onnx")
    assert res.returncode == 0, res.stderr[-2000:]
    first = O.import_net_from_onnx_bytes(data)
    assert [(l.kind, l.out_shape) for l in first.layers] == [(l.kind, l.out_shape) for l in net.layers]
    got = [l for l in res.stdout.splitlines() if l.startswith("layer ")]
    want = layer_lines(first)
    assert [g.split(" | ")[0] for g in got] == [w.split(" | ")[0] for w in want]
    second = O.import_net_from_onnx_file(str(tmp_path / "b.onnx"))
    assert [(l.kind, l.name, l.out_shape) for l in second.layers] == [(l.kind, l.name, l.out_shape) for l in first.layers]
    for a, b in zip(first.layers, second.layers):
        for key in a.params:
            if key == "bias" and not (a.attrs["cd"].use_bias if a.kind == "conv2d" else a.attrs.get("use_bias", True)):
                continue
            assert np.array_equal(a.params[key], b.params[key]), (a.name, key)
        if a.kind == "conv2d":
            assert (a.attrs["cd"].pads, a.attrs["cd"].sr) == (b.attrs["cd"].pads, b.attrs["cd"].sr)
        if a.kind == "pad":
            assert a.attrs["pads"] == b.attrs["pads"]
